#!/usr/bin/env python3
"""Benchmark of the row-wise operator kernels on one MI355X.

Default run (the line the driver records): the Llama-7B token shape —
RMSNorm forward + backward, bf16, 32768 packed tokens x hidden 4096, eps 1e-6.
One "step" is one forward + one backward over that batch, inputs resident in
HBM.  `value` is algorithmic GB/s of the whole step (every input read once,
every output written once).  The `roofline` object is for the dominant kernel
of the step (the backward row kernel), timed with HIP events recorded around
that kernel on its stream; `cpu_baseline` is the oracle's fp32 CPU port timed
on a bounded sample of the same rows.

Every run starts each measured case with an untimed pre-roll (PREROLL_* below) whatever
`--warmup` says: after idle the GPU's clocks take a few hundred launches to settle, and a
timed region that falls into the ramp reads 15 % slow.  The count is reported as
`preroll_steps`.

The line also carries `kernels`: every forward / backward kernel of every BASELINE
configuration (C1..C5) with its own microseconds, GB/s and fraction of the HBM peak over
KERNEL_STEPS launches, and `cpu_baselines`: the CPU ports of the reference's CPU kernels
for the same configurations on bounded samples.  `--all` adds the kernels beyond the
configurations, the streaming yardsticks and PyTorch-ROCm's own operators.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
IGNORE = -100
# untimed launches before any timed region of a case: at least this many and at least this long
PREROLL_MIN_STEPS = 300
PREROLL_MIN_SECONDS = 0.3
# timed launches per entry of the `kernels` table
KERNEL_STEPS = 200


def _load():
    import __graft_entry__
    __graft_entry__.ensure_built()      # a fresh checkout: compile once; built libraries are used as they are
    hk = importlib.import_module("hotspa-ae_amd")
    hk.lib()  # fails loudly when the HIP library is missing
    return hk


# ---------------------------------------------------------------------------
# cases: each builds `nsets` rotating buffer sets and returns (launch(i), bytes, rows, main-kernel name)
# ---------------------------------------------------------------------------
def _randn(torch, shape, dtype, std=1.0, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    n = 1
    for s in shape:
        n *= s
    out = torch.empty(shape, dtype=dtype, device="cuda")
    flat = out.view(-1)
    step = 1 << 26
    for o in range(0, n, step):  # chunked: no full-size fp32 temporary
        m = min(step, n - o)
        flat[o:o + m] = (torch.randn(m, generator=g, device="cuda", dtype=torch.float32) * std).to(dtype)
    return out


def _uniform(torch, shape, dtype, lo, hi, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.rand(shape, generator=g, device="cuda", dtype=torch.float32) * (hi - lo) + lo).to(dtype)


def case_rmsnorm(hk, torch, nsets, which):
    rows, cols, eps = 32768, 4096, 1e-6
    bf = torch.bfloat16
    sets = []
    for i in range(nsets):
        s = dict(x=_randn(torch, (rows, cols), bf, 1.0, 402 + 10 * i), dz=_randn(torch, (rows, cols), bf, 1.0, 404 + 10 * i),
                 z=torch.empty((rows, cols), dtype=bf, device="cuda"), dx=torch.empty((rows, cols), dtype=bf, device="cuda"),
                 mu=torch.empty(rows, device="cuda"), rs=torch.empty(rows, device="cuda"))
        sets.append(s)
    w = _uniform(torch, (cols,), bf, 0.8, 1.2, 403)
    dg, db = torch.empty_like(w), torch.empty_like(w)
    ws = torch.empty(max(1, hk.norm_bwd_workspace_bytes(8, rows, cols) // 4), device="cuda")
    for s in sets:
        hk.dropout_add_ln_fwd(s["x"], None, w, None, s["z"], None, s["mu"], s["rs"], eps, True)
    fwd_bytes = 2 * rows * cols * 2 + cols * 2 + rows * 4 + rows * 4
    bwd_bytes = 3 * rows * cols * 2 + rows * 4 + cols * 2 + cols * 2

    def fwd(i):
        s = sets[i % nsets]
        hk.dropout_add_ln_fwd(s["x"], None, w, None, s["z"], None, s["mu"], s["rs"], eps, True)

    def bwd(i):
        s = sets[i % nsets]
        # an RMSNorm has no bias: dx and dgamma are what its backward is asked for
        hk.dropout_add_ln_bwd(s["dz"], None, s["x"], s["mu"], s["rs"], w, s["dx"], None, dg, None, True, workspace=ws)

    if which == "fwd":
        return fwd, fwd_bytes, rows
    if which == "bwd":
        return bwd, bwd_bytes, rows
    return (lambda i: (fwd(i), bwd(i))), fwd_bytes + bwd_bytes, rows


def case_rmsnorm_pitched(hk, torch, nsets, which):
    """The headline shape as a column slice of a wider buffer: rows of 4096 bf16 columns lying 4608 apart, inputs and
    outputs alike.  The kernels take the pitch; nothing is copied."""
    rows, cols, wide, eps = 32768, 4096, 4608, 1e-6
    bf = torch.bfloat16
    sets = []
    for i in range(nsets):
        big = {k: torch.empty((rows, wide), dtype=bf, device="cuda") for k in ("x", "dz", "z", "dx")}
        big["x"][:, :cols] = _randn(torch, (rows, cols), bf, 1.0, 402 + 10 * i)
        big["dz"][:, :cols] = _randn(torch, (rows, cols), bf, 1.0, 404 + 10 * i)
        s = {k: v[:, 256:256 + cols] if k in ("z", "dx") else v[:, :cols] for k, v in big.items()}
        s["mu"], s["rs"] = torch.empty(rows, device="cuda"), torch.empty(rows, device="cuda")
        sets.append(s)
    w = _uniform(torch, (cols,), bf, 0.8, 1.2, 403)
    dg, db = torch.empty_like(w), torch.empty_like(w)
    ws = torch.empty(max(1, hk.norm_bwd_workspace_bytes(8, rows, cols) // 4), device="cuda")
    for s in sets:
        hk.dropout_add_ln_fwd(s["x"], None, w, None, s["z"], None, s["mu"], s["rs"], eps, True)
    if which == "fwd":
        return (lambda i: hk.dropout_add_ln_fwd(sets[i % nsets]["x"], None, w, None, sets[i % nsets]["z"], None,
                                                sets[i % nsets]["mu"], sets[i % nsets]["rs"], eps, True)), \
            2 * rows * cols * 2 + cols * 2 + rows * 8, rows
    return (lambda i: hk.dropout_add_ln_bwd(sets[i % nsets]["dz"], None, sets[i % nsets]["x"], sets[i % nsets]["mu"],
                                            sets[i % nsets]["rs"], w, sets[i % nsets]["dx"], None, dg, None, True,
                                            workspace=ws)), \
        3 * rows * cols * 2 + rows * 4 + cols * 2 + cols * 2, rows


def case_rmsnorm_permuted(hk, torch, nsets, which):
    """The headline shape as a view with permuted leading dimensions: arrays stored [2048, 16, 4096] (sequence first)
    and used as [16, 2048, 4096] (batch first) through permute(1, 0, 2), inputs and outputs alike.  Rows stay contiguous,
    the leading dimensions lie on two levels; the kernels take the steps, nothing is gathered or scattered."""
    S, B, cols, eps = 2048, 16, 4096, 1e-6
    rows = S * B
    bf = torch.bfloat16
    sets = []
    for i in range(nsets):
        st = {k: torch.empty((S, B, cols), dtype=bf, device="cuda") for k in ("x", "dz", "z", "dx")}
        st["x"].copy_(_randn(torch, (S, B, cols), bf, 1.0, 402 + 10 * i))
        st["dz"].copy_(_randn(torch, (S, B, cols), bf, 1.0, 404 + 10 * i))
        s = {k: v.permute(1, 0, 2) for k, v in st.items()}
        s["mu"], s["rs"] = torch.empty(rows, device="cuda"), torch.empty(rows, device="cuda")
        sets.append(s)
    w = _uniform(torch, (cols,), bf, 0.8, 1.2, 403)
    dg, db = torch.empty_like(w), torch.empty_like(w)
    ws = torch.empty(max(1, hk.norm_bwd_workspace_bytes(8, rows, cols) // 4), device="cuda")
    for s in sets:
        hk.dropout_add_ln_fwd(s["x"], None, w, None, s["z"], None, s["mu"], s["rs"], eps, True)
    if which == "fwd":
        return (lambda i: hk.dropout_add_ln_fwd(sets[i % nsets]["x"], None, w, None, sets[i % nsets]["z"], None,
                                                sets[i % nsets]["mu"], sets[i % nsets]["rs"], eps, True)), \
            2 * rows * cols * 2 + cols * 2 + rows * 8, rows
    return (lambda i: hk.dropout_add_ln_bwd(sets[i % nsets]["dz"], None, sets[i % nsets]["x"], sets[i % nsets]["mu"],
                                            sets[i % nsets]["rs"], w, sets[i % nsets]["dx"], None, dg, None, True,
                                            workspace=ws)), \
        3 * rows * cols * 2 + rows * 4 + cols * 2 + cols * 2, rows


def case_softmax_permuted(hk, torch, nsets, which):
    """Softmax over the last dimension of attention scores stored [4, 2048, 32, 2048] (batch, query, head, key) and used
    as [4, 32, 2048, 2048] through permute(0, 2, 1, 3): three levels of rows, read and written in place."""
    B, H, S = 4, 32, 2048
    bf = torch.bfloat16
    n = B * H * S * S
    sets = []
    for i in range(nsets):
        st = {k: torch.empty((B, S, H, S), dtype=bf, device="cuda") for k in ("x", "y", "dy", "dx")}
        st["x"].copy_(_randn(torch, (B, S, H, S), bf, 3.0, 201 + 10 * i))
        st["dy"].copy_(_randn(torch, (B, S, H, S), bf, 1.0, 202 + 10 * i))
        s = {k: v.permute(0, 2, 1, 3) for k, v in st.items()}
        hk.softmax_fwd(s["x"], s["y"])
        sets.append(s)
    if which == "fwd":
        return (lambda i: hk.softmax_fwd(sets[i % nsets]["x"], sets[i % nsets]["y"])), 2 * n * 2, B * H * S
    return (lambda i: hk.softmax_bwd(sets[i % nsets]["y"], sets[i % nsets]["dy"], sets[i % nsets]["dx"])), 3 * n * 2, B * H * S


def case_layernorm(hk, torch, nsets, which, cfg):
    if cfg == "C1":
        rows, cols, dt, eps = 8192, 4096, torch.float32, 1e-5
    else:
        rows, cols, dt, eps = 16384, 5120, torch.bfloat16, 1e-5
    es = 4 if dt == torch.float32 else 2
    sets = []
    for i in range(nsets):
        sets.append(dict(x=_randn(torch, (rows, cols), dt, 1.0, 101 + 10 * i), dy=_randn(torch, (rows, cols), dt, 1.0, 514 + 10 * i),
                         y=torch.empty((rows, cols), dtype=dt, device="cuda"), dx=torch.empty((rows, cols), dtype=dt, device="cuda"),
                         mean=torch.empty(rows, device="cuda"), rstd=torch.empty(rows, device="cuda")))
    g = _uniform(torch, (cols,), dt, 0.5, 1.5, 102)
    b = (_randn(torch, (cols,), torch.float32, 0.1, 103)).to(dt)
    dg, db = torch.empty_like(g), torch.empty_like(g)
    ws = torch.empty(max(1, hk.norm_bwd_workspace_bytes(hk.dtype_code(g), rows, cols) // 4), device="cuda")
    for s in sets:
        hk.layer_norm_fwd(s["x"], g, b, s["y"], s["mean"], s["rstd"], eps, stat_kind=1)
    fwd_bytes = 2 * rows * cols * es + 2 * cols * es + 2 * rows * 4
    bwd_bytes = 3 * rows * cols * es + 2 * rows * 4 + cols * es + 2 * cols * es

    def fwd(i):
        s = sets[i % nsets]
        hk.layer_norm_fwd(s["x"], g, b, s["y"], s["mean"], s["rstd"], eps, stat_kind=1)

    def bwd(i):
        s = sets[i % nsets]
        hk.layer_norm_bwd(s["dy"], s["x"], g, b, s["mean"], s["rstd"], s["dx"], dg, db, eps, stat_kind=1,
                          clamp_gamma=True, workspace=ws)

    return (fwd, fwd_bytes, rows) if which == "fwd" else (bwd, bwd_bytes, rows)


def case_softmax(hk, torch, nsets, which):
    shape = (4, 32, 2048, 2048)
    rows = 4 * 32 * 2048
    bf = torch.bfloat16
    sets = []
    for i in range(nsets):
        s = dict(x=_randn(torch, shape, bf, 3.0, 201 + 10 * i), y=torch.empty(shape, dtype=bf, device="cuda"))
        hk.softmax_fwd(s["x"], s["y"])
        if which == "bwd":
            s["dy"] = _randn(torch, shape, bf, 1.0, 202 + 10 * i)
            s["dx"] = s.pop("x")  # reuse the storage: x is not read by backward
        sets.append(s)
    n = rows * 2048 * 2
    if which == "fwd":
        return (lambda i: hk.softmax_fwd(sets[i % nsets]["x"], sets[i % nsets]["y"])), 2 * n, rows
    return (lambda i: hk.softmax_bwd(sets[i % nsets]["y"], sets[i % nsets]["dy"], sets[i % nsets]["dx"])), 3 * n, rows


def case_sce(hk, torch, nsets, which):
    rows, cols = 16384, 32000
    bf = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(502)
    labels = torch.randint(0, cols, (rows,), generator=g, device="cuda", dtype=torch.int64)
    drop = torch.rand(rows, generator=g, device="cuda") < 0.05
    labels[drop] = IGNORE
    sets = []
    for i in range(nsets):
        s = dict(x=_randn(torch, (rows, cols), bf, 2.0, 501 + 10 * i))
        if which == "bwd":
            s["dx"] = torch.empty((rows, cols), dtype=bf, device="cuda")
        sets.append(s)
    loss = torch.empty(rows, dtype=bf, device="cuda")
    gl = torch.full((rows,), 1.0 / rows, dtype=bf, device="cuda")
    n = rows * cols * 2
    # rows whose label is the ignored index are not read (their loss is 0, their gradient row is zeros): the bytes
    # really moved are the algorithmic ones less one logits row per such row
    ignored = int(drop.sum().item())
    if which == "fwd":
        launch = lambda i: hk.sce_sparse_fwd(sets[i % nsets]["x"], labels, loss, IGNORE)
        nbytes = n + rows * 8 + rows * 2
    else:
        launch = lambda i: hk.sce_sparse_bwd(sets[i % nsets]["x"], labels, gl, sets[i % nsets]["dx"], IGNORE)
        nbytes = 2 * n + rows * 8 + rows * 2
    launch.bytes_moved = nbytes - ignored * cols * 2
    launch.ignored_rows = ignored
    return launch, nbytes, rows


def case_nll_bwd(hk, torch, nsets):
    rows, cols = 16384, 32000
    bf = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(602)
    labels = torch.randint(0, cols, (rows,), generator=g, device="cuda", dtype=torch.int64)
    gl = torch.full((rows,), 1.0 / rows, dtype=bf, device="cuda")
    outs = [torch.empty((rows, cols), dtype=bf, device="cuda") for _ in range(2)]
    return (lambda i: hk.nll_loss_bwd(labels, gl, outs[i % 2])), rows * cols * 2 + rows * 10, rows


def case_instance_norm(hk, torch, nsets):
    # [N=256, C=256, H=32, W=32] bf16: 65536 planes of 1024 elements, no scale / bias
    rows, cols = 256 * 256, 32 * 32
    bf = torch.bfloat16
    xs = [_randn(torch, (rows, cols), bf, 1.0, 611 + i) for i in range(nsets)]
    ys = [torch.empty((rows, cols), dtype=bf, device="cuda") for _ in range(nsets)]
    mean = torch.empty(rows, dtype=bf, device="cuda")
    var = torch.empty(rows, dtype=bf, device="cuda")
    return (lambda i: hk.layer_norm_fwd(xs[i % nsets], None, None, ys[i % nsets], mean, var, 1e-5, stat_kind=0)), \
        2 * rows * cols * 2 + 2 * rows * 2, rows


def case_dropout_ln(hk, torch, nsets, which):
    """Pre-norm residual block at the headline shape: x = dropout(x0, 0.1) + residual, z = RMSNorm(x); the
    backward takes the gradients of z and of the residual stream and returns those of x0 and the residual."""
    rows, cols, eps, p = 32768, 4096, 1e-6, 0.1
    bf = torch.bfloat16
    n = rows * cols
    sets = []
    for i in range(nsets):
        s = dict(x0=_randn(torch, (rows, cols), bf, 1.0, 702 + 10 * i), res=_randn(torch, (rows, cols), bf, 1.0, 703 + 10 * i),
                 z=torch.empty((rows, cols), dtype=bf, device="cuda"), x=torch.empty((rows, cols), dtype=bf, device="cuda"),
                 m=torch.empty((rows, cols), dtype=torch.uint8, device="cuda"),
                 mu=torch.empty(rows, device="cuda"), rs=torch.empty(rows, device="cuda"))
        sets.append(s)
    w = _uniform(torch, (cols,), bf, 0.8, 1.2, 704)
    dg, db = torch.empty_like(w), torch.empty_like(w)

    def fwd(i):
        s = sets[i % nsets]
        hk.dropout_add_ln_fwd_ex(s["x0"], w, s["z"], s["mu"], s["rs"], residual=s["res"], x=s["x"], dmask=s["m"],
                                 dropout_p=p, eps=eps, is_rms=True, seed=1234, offset=i)

    for i in range(nsets):
        fwd(i)
    if which == "fwd":
        return fwd, n * (2 + 2 + 2 + 2 + 1) + cols * 2 + rows * 8, rows
    # backward reuses x0 / res storage for its outputs (they are not read by it)
    dz = [_randn(torch, (rows, cols), bf, 1.0, 705 + 10 * i) for i in range(nsets)]
    ws = hk.dropout_add_ln_bwd_ex(dz[0], sets[0]["x"], sets[0]["mu"], sets[0]["rs"], w, sets[0]["x0"], dx=sets[0]["z"],
                                  dmask=sets[0]["m"], dresidual=sets[0]["res"], dgamma=dg, dbeta=db, dropout_p=p,
                                  is_rms=True)

    def bwd(i):
        s = sets[i % nsets]
        hk.dropout_add_ln_bwd_ex(dz[i % nsets], s["x"], s["mu"], s["rs"], w, s["x0"], dx=s["z"], dmask=s["m"],
                                 dresidual=s["res"], dgamma=dg, dbeta=db, dropout_p=p, is_rms=True, workspace=ws)
    return bwd, n * (2 + 2 + 2 + 1 + 2 + 2) + rows * 4 + cols * 6, rows


def case_elementwise(hk, torch, nsets, which):
    """Steps of the vocabulary-parallel loss on one shard of [16384 x 32000] bf16 logits: logits - row maximum
    (per-row operand), exp in place, softmax = exp / row sum in place, and the gradient kernel."""
    rows, cols = 16384, 32000
    bf = torch.bfloat16
    n = rows * cols
    xs = [_randn(torch, (rows, cols), bf, 2.0, 801 + i) for i in range(2)]
    outs = [torch.empty((rows, cols), dtype=bf, device="cuda") for _ in range(2)]
    per_row = _uniform(torch, (rows, 1), bf, 1.0, 2.0, 811)
    if which == "sub":
        return (lambda i: hk.binary("sub", xs[i % 2], per_row, outs[i % 2])), 2 * n * 2 + rows * 2, rows
    if which == "exp":
        return (lambda i: hk.unary("exp", xs[i % 2], outs[i % 2])), 2 * n * 2, rows
    if which == "add":   # two dense operands of the same shape: the commonest element-wise call
        return (lambda i: hk.binary("add", xs[i % 2], outs[(i + 1) % 2], outs[i % 2])), 3 * n * 2, rows
    if which == "div":
        return (lambda i: hk.binary("div", xs[i % 2], per_row, xs[i % 2])), 2 * n * 2 + rows * 2, rows
    g = torch.Generator(device="cuda").manual_seed(812)
    labels = torch.randint(0, 4 * cols, (rows,), generator=g, device="cuda", dtype=torch.int64)
    gl = torch.full((rows,), 1.0 / rows, dtype=bf, device="cuda")
    if which == "vce":
        return (lambda i: hk.vocab_parallel_ce_bwd(xs[i % 2], labels, gl, outs[i % 2], cols)), 2 * n * 2 + rows * 10, rows
    # the fused form: shard 1 of 4 (columns [32000, 64000))
    stats = torch.empty(3, rows, device="cuda")
    if which == "stats":
        return (lambda i: hk.vocab_parallel_ce_stats(xs[i % 2], labels, stats, cols, IGNORE)), n * 2 + rows * 20, rows
    lse = torch.full((rows,), 12.0, device="cuda")
    return (lambda i: hk.vocab_parallel_ce_bwd_fused(xs[i % 2], labels, lse, gl, outs[i % 2], cols, IGNORE)), \
        2 * n * 2 + rows * 14, rows


def case_batch_norm(hk, torch, nsets, which):
    """Spatial batch norm in training mode, bf16 [256, 256, 56, 56]: statistics pass + element-wise pass
    (forward: x read twice, y written once; backward: dy and x read twice, dx written once)."""
    shape = (256, 256, 56, 56)
    bf = torch.bfloat16
    n = 256 * 256 * 56 * 56
    xs = [_randn(torch, shape, bf, 1.5, 821 + i) for i in range(2)]
    ys = [torch.empty(shape, dtype=bf, device="cuda") for _ in range(2)]
    scale = _uniform(torch, (256,), torch.float32, 0.5, 1.5, 822)
    bias = _randn(torch, (256,), torch.float32, 1.0, 823)
    rm, rv = torch.zeros(256, device="cuda"), torch.ones(256, device="cuda")
    sm, si = torch.empty(256, device="cuda"), torch.empty(256, device="cuda")
    ws = torch.empty(hk.batch_norm_workspace_bytes(xs[0]) // 4 + 4, device="cuda")
    hk.batch_norm_fwd(xs[0], scale, bias, ys[0], 0.1, 1e-5, rm, rv, sm, si, workspace=ws)
    if which == "fwd":
        def launch(i):
            hk.batch_norm_fwd(xs[i % 2], scale, bias, ys[i % 2], 0.1, 1e-5, rm, rv, sm, si, workspace=ws)
        launch.main_bytes = 2 * n * 2      # the element-wise pass alone: x read, y written
        return launch, 3 * n * 2, 256
    dys = [_randn(torch, shape, bf, 1.0, 825 + i) for i in range(2)]
    ds, db = torch.empty(256, device="cuda"), torch.empty(256, device="cuda")

    def launch(i):
        hk.batch_norm_bwd(dys[i % 2], xs[i % 2], scale, ys[i % 2], ds, db, sm, si, workspace=ws)
    launch.main_bytes = 3 * n * 2          # the element-wise pass alone: dy and x read, dx written
    return launch, 5 * n * 2, 256


def case_reduce(hk, torch, nsets, axes, op, three_d=False):
    rows, cols = 32768, 4096
    bf = torch.bfloat16
    sets = [_randn(torch, (rows, cols), bf, 1.0, 301 + 10 * i) for i in range(nsets)]
    if three_d:
        sets = [t.view(64, 512, 4096) for t in sets]
    nout = cols if 0 in axes else rows
    out = torch.empty(nout, dtype=bf, device="cuda")
    shape, strides = list(sets[0].shape), list(sets[0].stride())
    ws = torch.empty(max(1, hk.reduce_workspace_bytes(8, shape, strides, list(axes)) // 4), device="cuda")
    return (lambda i: hk.reduce(sets[i % nsets], out, list(axes), op, workspace=ws)), rows * cols * 2 + nout * 2, \
        (rows if 1 in axes and not three_d else cols)


def case_p_norm(hk, torch, nsets, which):
    """2-norm of every row of a bf16 [32768 x 4096] array (read only), and its gradient (2 reads, 1 write)."""
    rows, cols = 32768, 4096
    bf = torch.bfloat16
    sets = [_randn(torch, (rows, cols), bf, 1.0, 901 + 10 * i) for i in range(nsets)]
    out = torch.empty(rows, dtype=bf, device="cuda")
    if which == "fwd":
        ws = torch.empty(max(1, hk.reduce_workspace_bytes(8, [rows, cols], [cols, 1], [1]) // 4), device="cuda")
        return (lambda i: hk.norm(sets[i % nsets], out, 1, 2, workspace=ws)), rows * cols * 2 + rows * 2, rows
    hk.norm(sets[0], out, 1, 2)
    grad = _randn(torch, (rows,), bf, 1.0, 977)
    dx = [torch.empty_like(t) for t in sets]
    return (lambda i: hk.norm_bwd(sets[i % nsets], out, grad, dx[i % nsets], 1, 2)), \
        2 * rows * cols * 2 + 2 * rows * 2, rows


def case_reduce_gradient(hk, torch, nsets, axis):
    """Gradient of a mean over `axis` of a bf16 [32768 x 4096] array: the output's gradient laid back over the
    input, times 1/n (write only but for one small vector)."""
    rows, cols = 32768, 4096
    bf = torch.bfloat16
    nin = cols if axis == 0 else rows
    grad = _randn(torch, (1, cols) if axis == 0 else (rows, 1), bf, 1.0, 951)
    outs = [torch.empty(rows, cols, dtype=bf, device="cuda") for _ in range(nsets)]
    scale = 1.0 / (rows if axis == 0 else cols)
    return (lambda i: hk.broadcast(grad, outs[i % nsets], scalar=scale)), rows * cols * 2 + nin * 2, rows


def case_copy(hk, torch, nsets):
    n = 1 << 28
    src = [torch.empty(n, dtype=torch.uint8, device="cuda").zero_() for _ in range(nsets)]
    dst = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(nsets)]
    return (lambda i: hk.copy_kernel(dst[i % nsets], src[i % nsets])), 2 * n, 1


def case_strided(hk, torch, nsets, which):
    """The extra pass an operator pays for an operand that is neither dense nor row-pitched: a permuted view gathered
    into a dense array (hk_strided_copy), or a dense result laid over such a view (hk_strided_scatter)."""
    if which == "transposed fp32":
        shape, perm, dt = (8192, 4096), (1, 0), torch.float32
    elif which == "swapped bf16":
        shape, perm, dt = (32, 2048, 2048), (0, 2, 1), torch.bfloat16
    else:   # rows stay contiguous: [64, 512, 4096] with the first two dimensions swapped
        shape, perm, dt = (64, 512, 4096), (1, 0, 2), torch.bfloat16
    srcs = [_randn(torch, shape, dt, 1.0, 961 + k) for k in range(nsets)]
    views = [x.permute(perm) for x in srcs]
    outs = [torch.empty(views[0].shape, dtype=dt, device="cuda") for _ in range(nsets)]
    nbytes = 2 * srcs[0].numel() * srcs[0].element_size()
    return (lambda i: hk.strided_copy(views[i % nsets], outs[i % nsets])), nbytes, 1


def case_fill(hk, torch, nsets):
    import ctypes
    n = 1 << 28
    dst = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(nsets)]
    lib = hk.lib()

    def launch(i):
        hk.check(lib.hk_memset(ctypes.c_void_p(dst[i % nsets].data_ptr()), ctypes.c_int(0), ctypes.c_size_t(n),
                               hk.current_stream()))
    return launch, n, 1


def case_torch_op(hk, torch, nsets, which):
    """PyTorch-ROCm's own operators at the benchmark shapes on the same GPU (its kernels for these ops are the
    CUDA sources compiled for AMD): yardsticks, not product paths.  Wall time per call, PyTorch's dispatch and
    autograd bookkeeping included; bytes counted as for this library's kernels."""
    F = torch.nn.functional
    bf = torch.bfloat16
    if which in ("rms_fwd", "rms_fwd_bwd"):
        rows, cols = 32768, 4096
        xs = [_randn(torch, (rows, cols), bf, 1.0, 401 + i).requires_grad_(True) for i in range(nsets)]
        dz = _randn(torch, (rows, cols), bf, 1.0, 499)
        w = _uniform(torch, (cols,), bf, 0.8, 1.2, 403).requires_grad_(True)
        if which == "rms_fwd":
            def launch(i):
                with torch.no_grad():
                    F.rms_norm(xs[i % nsets], (cols,), w, 1e-6)
            nbytes = rows * (2 * cols * 2 + 4) + cols * 2
        else:
            def launch(i):
                z = F.rms_norm(xs[i % nsets], (cols,), w, 1e-6)
                torch.autograd.grad(z, (xs[i % nsets], w), dz)
            nbytes = rows * (5 * cols * 2 + 12)
        units = rows
    elif which in ("softmax_fwd", "softmax_bwd"):
        shape = (4, 32, 2048, 2048)
        n = 4 * 32 * 2048 * 2048
        xs = [_randn(torch, shape, bf, 1.0, 201 + i) for i in range(2)]
        if which == "softmax_fwd":
            def launch(i):
                torch.softmax(xs[i % 2], -1)
            nbytes = 2 * n * 2
        else:
            ys = [torch.softmax(x, -1) for x in xs]
            dy = _randn(torch, shape, bf, 1.0, 299)

            def launch(i):
                torch._softmax_backward_data(dy, ys[i % 2], -1, bf)
            nbytes = 3 * n * 2
        units = n // 2048
    elif which in ("ln_fwd_c1", "ln_fwd_bwd_c5"):
        if which == "ln_fwd_c1":
            rows, cols, dt = 8192, 4096, torch.float32
        else:
            rows, cols, dt = 16384, 5120, bf
        es = 4 if dt == torch.float32 else 2
        xs = [_randn(torch, (rows, cols), dt, 1.0, 101 + i).requires_grad_(True) for i in range(nsets)]
        w = _uniform(torch, (cols,), dt, 0.5, 1.5, 103).requires_grad_(True)
        b = _randn(torch, (cols,), dt, 0.1, 104).requires_grad_(True)
        if which == "ln_fwd_c1":
            def launch(i):
                with torch.no_grad():
                    F.layer_norm(xs[i % nsets], (cols,), w, b, 1e-5)
            nbytes = rows * (2 * cols * es + 8) + 2 * cols * es
        else:
            dz = _randn(torch, (rows, cols), dt, 1.0, 199)

            def launch(i):
                z = F.layer_norm(xs[i % nsets], (cols,), w, b, 1e-5)
                torch.autograd.grad(z, (xs[i % nsets], w, b), dz)
            nbytes = rows * (5 * cols * es + 16)
        units = rows
    elif which in ("sum_axis0", "sum_axis1"):
        rows, cols = 32768, 4096
        xs = [_randn(torch, (rows, cols), bf, 1.0, 301 + 10 * i) for i in range(nsets)]
        axis = 0 if which == "sum_axis0" else 1

        def launch(i):
            torch.sum(xs[i % nsets], dim=axis)
        nbytes = rows * cols * 2 + (cols if axis == 0 else rows) * 2
        units = rows
    else:
        rows, cols = 16384, 32000
        xs = [_randn(torch, (rows, cols), bf, 2.0, 501 + i).requires_grad_(True) for i in range(2)]
        g = torch.Generator(device="cuda").manual_seed(77)
        labels = torch.randint(0, cols, (rows,), generator=g, device="cuda")
        labels[::20] = -100
        if which == "ce_fwd":
            def launch(i):
                with torch.no_grad():
                    F.cross_entropy(xs[i % 2], labels, ignore_index=-100)
            nbytes = rows * (cols * 2 + 8 + 2)
        else:
            def launch(i):
                loss = F.cross_entropy(xs[i % 2], labels, ignore_index=-100)
                torch.autograd.grad(loss, xs[i % 2])
            nbytes = rows * (3 * cols * 2 + 2 * (8 + 2))
        units = rows
    launch.no_hook = True
    return launch, nbytes, units


def case_torch_add(hk, torch, nsets):
    """torch's own elementwise add (two reads, one write per element): an independent yardstick for what
    a plain streaming kernel with this read/write mix reaches on the same GPU."""
    rows, cols = 32768, 4096
    bf = torch.bfloat16
    a = [_randn(torch, (rows, cols), bf, 1.0, 901 + i) for i in range(nsets)]
    b = [_randn(torch, (rows, cols), bf, 1.0, 951 + i) for i in range(nsets)]
    o = [torch.empty((rows, cols), dtype=bf, device="cuda") for _ in range(nsets)]

    def launch(i):
        torch.add(a[i % nsets], b[i % nsets], out=o[i % nsets])
    launch.no_hook = True
    return launch, 3 * rows * cols * 2, rows


def is_config_case(name):
    """The kernels of the BASELINE configurations: always measured, also by the default run."""
    return name[:2] in ("C1", "C2", "C3", "C4", "C5")


CASES = [
    ("C1 layernorm fwd fp32 [8192x4096]", lambda hk, t, n: case_layernorm(hk, t, n, "fwd", "C1")),
    ("C2 softmax fwd bf16 [4,32,2048,2048]", lambda hk, t, n: case_softmax(hk, t, 2, "fwd")),
    ("C2 softmax bwd bf16 [4,32,2048,2048]", lambda hk, t, n: case_softmax(hk, t, 2, "bwd")),
    ("C3 reduce sum axis0 bf16 [32768x4096]", lambda hk, t, n: case_reduce(hk, t, n, (0,), "sum")),
    ("C3 reduce mean axis0 bf16 [32768x4096]", lambda hk, t, n: case_reduce(hk, t, n, (0,), "mean")),
    ("C3 reduce sum axis1 bf16 [32768x4096]", lambda hk, t, n: case_reduce(hk, t, n, (1,), "sum")),
    ("C3 reduce mean axis1 bf16 [32768x4096]", lambda hk, t, n: case_reduce(hk, t, n, (1,), "mean")),
    ("C3 reduce sum axes(0,1) bf16 [64x512x4096]", lambda hk, t, n: case_reduce(hk, t, n, (0, 1), "sum", True)),
    ("next: rmsnorm fwd bf16 on a [32768x4096] slice of [32768x4608] (row-pitched in and out)",
     lambda hk, t, n: case_rmsnorm_pitched(hk, t, n, "fwd")),
    ("next: rmsnorm bwd bf16 on a [32768x4096] slice of [32768x4608] (row-pitched in and out)",
     lambda hk, t, n: case_rmsnorm_pitched(hk, t, n, "bwd")),
    ("next: rmsnorm fwd bf16 on a [16,2048,4096] view of a [2048,16,4096] array (leading dimensions permuted, in and out)",
     lambda hk, t, n: case_rmsnorm_permuted(hk, t, n, "fwd")),
    ("next: rmsnorm bwd bf16 on a [16,2048,4096] view of a [2048,16,4096] array (leading dimensions permuted, in and out)",
     lambda hk, t, n: case_rmsnorm_permuted(hk, t, n, "bwd")),
    ("next: softmax fwd bf16 on a [4,32,2048,2048] view of a [4,2048,32,2048] array (leading dimensions permuted, in and out)",
     lambda hk, t, n: case_softmax_permuted(hk, t, 2, "fwd")),
    ("next: softmax bwd bf16 on a [4,32,2048,2048] view of a [4,2048,32,2048] array (leading dimensions permuted, in and out)",
     lambda hk, t, n: case_softmax_permuted(hk, t, 2, "bwd")),
    ("next: reduce max axis0 bf16 [32768x4096]", lambda hk, t, n: case_reduce(hk, t, n, (0,), "max")),
    ("next: reduce max axis1 bf16 [32768x4096]", lambda hk, t, n: case_reduce(hk, t, n, (1,), "max")),
    ("next: reduce prod axis1 bf16 [32768x4096]", lambda hk, t, n: case_reduce(hk, t, n, (1,), "prod")),
    ("next: nll loss bwd bf16 [16384x32000] (write only)", lambda hk, t, n: case_nll_bwd(hk, t, n)),
    ("next: instance norm fwd bf16 [256,256,32,32]", lambda hk, t, n: case_instance_norm(hk, t, n)),
    ("next: dropout(0.1)+residual+rmsnorm fwd bf16 [32768x4096]", lambda hk, t, n: case_dropout_ln(hk, t, 2, "fwd")),
    ("next: dropout(0.1)+residual+rmsnorm bwd bf16 [32768x4096]", lambda hk, t, n: case_dropout_ln(hk, t, 2, "bwd")),
    ("next: logits - row max bf16 [16384x32000]", lambda hk, t, n: case_elementwise(hk, t, n, "sub")),
    ("next: dense + dense bf16 [16384x32000] (2R:1W)", lambda hk, t, n: case_elementwise(hk, t, n, "add")),
    ("next: exp bf16 [16384x32000]", lambda hk, t, n: case_elementwise(hk, t, n, "exp")),
    ("next: exp / row sum in place bf16 [16384x32000]", lambda hk, t, n: case_elementwise(hk, t, n, "div")),
    ("next: vocab-parallel CE bwd bf16 [16384x32000]", lambda hk, t, n: case_elementwise(hk, t, n, "vce")),
    ("next: vocab-parallel CE fused stats bf16 [16384x32000] (read only)", lambda hk, t, n: case_elementwise(hk, t, n, "stats")),
    ("next: vocab-parallel CE fused bwd bf16 [16384x32000]", lambda hk, t, n: case_elementwise(hk, t, n, "fused")),
    ("next: 2-norm of rows bf16 [32768x4096] (read only)", lambda hk, t, n: case_p_norm(hk, t, n, "fwd")),
    ("next: 2-norm of rows, gradient bf16 [32768x4096]", lambda hk, t, n: case_p_norm(hk, t, n, "bwd")),
    ("next: gradient of mean axis0 bf16 [32768x4096] (write only)", lambda hk, t, n: case_reduce_gradient(hk, t, n, 0)),
    ("next: gradient of mean axis1 bf16 [32768x4096] (write only)", lambda hk, t, n: case_reduce_gradient(hk, t, n, 1)),
    ("next: batch norm fwd bf16 [256,256,56,56] (2R+1W, 3 launches)", lambda hk, t, n: case_batch_norm(hk, t, n, "fwd")),
    ("next: batch norm bwd bf16 [256,256,56,56] (4R+1W, 3 launches)", lambda hk, t, n: case_batch_norm(hk, t, n, "bwd")),
    ("next: gather of a transposed view fp32 [8192x4096]", lambda hk, t, n: case_strided(hk, t, n, "transposed fp32")),
    ("next: gather of a view with the last two dimensions swapped bf16 [32x2048x2048]",
     lambda hk, t, n: case_strided(hk, t, n, "swapped bf16")),
    ("next: gather of a view with the first two dimensions swapped bf16 [64x512x4096]",
     lambda hk, t, n: case_strided(hk, t, n, "outer bf16")),
    ("C4 rmsnorm fwd bf16 [32768x4096]", lambda hk, t, n: case_rmsnorm(hk, t, n, "fwd")),
    ("C4 rmsnorm bwd bf16 [32768x4096]", lambda hk, t, n: case_rmsnorm(hk, t, n, "bwd")),
    ("C5 sce fwd bf16 [16384x32000]", lambda hk, t, n: case_sce(hk, t, 2, "fwd")),
    ("C5 sce bwd bf16 [16384x32000]", lambda hk, t, n: case_sce(hk, t, 2, "bwd")),
    ("C5 layernorm fwd bf16 [16384x5120]", lambda hk, t, n: case_layernorm(hk, t, n, "fwd", "C5")),
    ("C5 layernorm bwd bf16 [16384x5120]", lambda hk, t, n: case_layernorm(hk, t, n, "bwd", "C5")),
    ("copy kernel 256 MiB (calibration)", lambda hk, t, n: case_copy(hk, t, n)),
    ("fill kernel 256 MiB (write-only calibration)", lambda hk, t, n: case_fill(hk, t, n)),
    ("torch.add bf16 [32768x4096] (2R:1W yardstick)", lambda hk, t, n: case_torch_add(hk, t, n)),
    ("torch F.rms_norm fwd bf16 [32768x4096] (yardstick for C4 fwd)", lambda hk, t, n: case_torch_op(hk, t, n, "rms_fwd")),
    ("torch F.rms_norm fwd+bwd bf16 [32768x4096] (yardstick for the headline)", lambda hk, t, n: case_torch_op(hk, t, n, "rms_fwd_bwd")),
    ("torch F.layer_norm fwd fp32 [8192x4096] (yardstick for C1)", lambda hk, t, n: case_torch_op(hk, t, n, "ln_fwd_c1")),
    ("torch F.layer_norm fwd+bwd bf16 [16384x5120] (yardstick for C5 LN fwd+bwd)", lambda hk, t, n: case_torch_op(hk, t, n, "ln_fwd_bwd_c5")),
    ("torch.sum axis0 bf16 [32768x4096] (yardstick for C3)", lambda hk, t, n: case_torch_op(hk, t, n, "sum_axis0")),
    ("torch.sum axis1 bf16 [32768x4096] (yardstick for C3)", lambda hk, t, n: case_torch_op(hk, t, n, "sum_axis1")),
    ("torch softmax fwd bf16 [4,32,2048,2048] (yardstick for C2 fwd)", lambda hk, t, n: case_torch_op(hk, t, n, "softmax_fwd")),
    ("torch softmax bwd bf16 [4,32,2048,2048] (yardstick for C2 bwd)", lambda hk, t, n: case_torch_op(hk, t, n, "softmax_bwd")),
    ("torch F.cross_entropy fwd bf16 [16384x32000] (yardstick for C5 fwd)", lambda hk, t, n: case_torch_op(hk, t, n, "ce_fwd")),
    ("torch F.cross_entropy fwd+bwd bf16 [16384x32000] (yardstick for C5 fwd+bwd)", lambda hk, t, n: case_torch_op(hk, t, n, "ce_fwd_bwd")),
]


# HBM bytes one launch of the RMSNorm backward kernel moves at the headline shape: rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE read 262834.3 and 266598.8 KiB per dispatch; a 256 MiB copy kernel calibrates the counters at
# x1.99993 (FETCH_SIZE reads 131076.5 KiB for 262144 KiB fetched) and x1.00000 (WRITE_SIZE reads 262145.9).
NORM_BWD_TRAFFIC_BYTES = int((262834.3 * 1.99993 + 266598.8 * 1.0) * 1024)


def preroll(torch, launch, min_steps=PREROLL_MIN_STEPS, min_seconds=PREROLL_MIN_SECONDS):
    """Untimed launches of the case until the clocks have settled; returns how many were made."""
    done, t0 = 0, time.perf_counter()
    while done < min_steps or time.perf_counter() - t0 < min_seconds:
        for _ in range(50):
            launch(done)
            done += 1
        torch.cuda.synchronize()
    return done


def time_case(hk, torch, launch, steps, warmup, profile_main=True):
    """Returns (ms per step over a plain timed region, mean us of the main kernel measured in a
    second region with HIP events recorded around that kernel on its stream, pre-roll launches made)."""
    pre = preroll(torch, launch)
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        launch(i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    main_us = None
    if profile_main:
        pairs = [(hk.Event(), hk.Event()) for _ in range(steps)]
        for i in range(steps):
            hk.check(hk.lib().hk_profile_next_kernel(pairs[i][0].h, pairs[i][1].h))
            launch(i)
        torch.cuda.synchronize()
        hk.lib().hk_profile_next_kernel(None, None)
        main_us = sum(b.elapsed_ns_since(a) for a, b in pairs) / 1000.0 / steps
    return (t1 - t0) * 1000.0 / steps, main_us, pre


def _cpu_cores():
    return min(int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1), 64)


def _timed_cpu(fn, budget_s):
    fn()                                    # pages the outputs in, warms whatever the call warms
    reps, t0 = 0, time.perf_counter()
    while reps < 2 or time.perf_counter() - t0 < budget_s:
        fn()
        reps += 1
    return (time.perf_counter() - t0) / reps, reps


def cpu_baseline(rows=32768, cols=4096, budget_s=2.0):
    """The headline step on the host: `value` is the fp32 CPU port of it (oracle's refcpu_rmsnorm_*) on all host
    threads over the full workload, repeated for about `budget_s` seconds; beside it the same port on ONE thread (the
    reference's scalar loops are serial and its build never enables OpenMP, CMakeLists.txt:33-36) on a quarter of the
    rows, and torch's own CPU operators (F.rms_norm and its autograd; MKL / oneDNN-class kernels) on all threads."""
    import ctypes
    import numpy as np
    import oracle
    lib = oracle.lib()
    cores = _cpu_cores()
    g = np.random.default_rng(402)
    # a 1024-row random block repeated down the array: the values do not change the timing
    reps_of_block = (rows + 1023) // 1024
    x = np.tile(g.standard_normal((1024, cols), dtype=np.float32), (reps_of_block, 1))[:rows].copy()
    dz = np.tile(g.standard_normal((1024, cols), dtype=np.float32), (reps_of_block, 1))[:rows].copy()
    w = (g.random(cols, dtype=np.float32) * 0.4 + 0.8).astype(np.float32)
    z = np.empty_like(x); dx = np.empty_like(x); rs = np.empty(rows, dtype=np.float32)
    dg = np.empty(cols, dtype=np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    P = lambda a: a.ctypes.data_as(fp)

    def step(n):
        lib.refcpu_rmsnorm_fwd_f32(P(x), P(w), ctypes.c_int64(n), ctypes.c_int64(cols), ctypes.c_float(1e-6), P(z), P(rs))
        lib.refcpu_rmsnorm_bwd_f32(P(dz), P(x), P(w), P(rs), ctypes.c_int64(n), ctypes.c_int64(cols), P(dx), P(dg))

    per_row = 5 * cols * 2 + 12             # same bf16 accounting as the GPU step
    lib.refcpu_set_num_threads(ctypes.c_int(cores))
    dt, reps = _timed_cpu(lambda: step(rows), budget_s)
    out = {"value": round(rows * per_row / dt / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
           "sample": "all %d rows, fwd+bwd in fp32, %d repetitions over %.1f s, mean; bytes counted as for the GPU step "
                     "(bf16 storage); RMSNorm has no CPU kernel in the reference, this is the oracle's fp32 port of the "
                     "formula" % (rows, reps, reps * dt)}
    # one thread, a quarter of the rows
    lib.refcpu_set_num_threads(ctypes.c_int(1))
    n1 = rows // 4
    dt1, reps1 = _timed_cpu(lambda: step(n1), 1.0)
    lib.refcpu_set_num_threads(ctypes.c_int(cores))
    out["one_thread"] = {"value": round(n1 * per_row / dt1 / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                         "sample": "%d of %d rows, %d repetitions, mean" % (n1, rows, reps1)}
    # torch's CPU operators on the same shape in bf16 (forward, then forward + backward through autograd)
    import torch
    torch.set_num_threads(cores)
    nt = rows // 16
    tx = torch.from_numpy(x[:nt]).to(torch.bfloat16).requires_grad_(True)
    tdz = torch.from_numpy(dz[:nt]).to(torch.bfloat16)
    tw = torch.from_numpy(w).to(torch.bfloat16).requires_grad_(True)

    def torch_step():
        tx.grad = None
        tw.grad = None
        torch.nn.functional.rms_norm(tx, (cols,), tw, 1e-6).backward(tdz)

    dtt, repst = _timed_cpu(torch_step, 1.0)
    out["torch_cpu"] = {"value": round(nt * per_row / dtt / 1e9, 3), "unit": "GB/s", "cores": cores,
                        "kind": "torch-cpu (oneDNN-class)",
                        "sample": "F.rms_norm forward + autograd backward, bf16, %d of %d rows, %d repetitions, mean"
                                  % (nt, rows, repst)}
    return out


def cpu_baselines(budget_s=0.5):
    """Per BASELINE configuration kernel, three host figures on a bounded sample of the configuration's rows (at least
    128 MB of input each, so that the sample does not sit in the last-level cache), in the configuration's storage
    type, counting the same algorithmic bytes per row as the GPU entry:
      * kind "port": the host twin of the kernel (LayerNormCpu / LayerNormGradientCpu, SoftmaxCpu / SoftmaxGradientCpu,
        SoftmaxCrossEntropySparseCpu / ...GradientCpu, ReduceCpu: the reference's CPU pass structure as fp32 loops,
        OpenMP over rows), called through the same operator entry points and device dispatch as the accelerator
        kernels, on all host threads;
      * kind "port (1 thread)": the same on one thread -- the reference's own scalar loops are serial and its build
        never enables OpenMP (CMakeLists.txt:33-36);
      * kind "torch-cpu (oneDNN-class)": torch's CPU operator of the same mathematics on all threads (MKL / oneDNN
        inside), standing in for the oneDNN primitives the reference calls (hetu/impl/kernel/Softmax.cc:31-45,
        Reduce.cc:41-68, LayerNorm.cc:89-129), whose library is not part of the reference's sources."""
    import importlib
    import torch
    import torch.nn.functional as F
    importlib.import_module("hotspa-ae_amd")
    ops = importlib.import_module("hotspa-ae_amd.hetu_ops")
    cores = _cpu_cores()
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(7)
    bf = torch.bfloat16

    def block(rows, cols, dt):
        b = torch.randn(min(rows, 512), cols, generator=g)
        return b.repeat((rows + b.shape[0] - 1) // b.shape[0], 1)[:rows].to(dt).contiguous()

    out = []

    def add(config, case, port_fn, torch_fn, algo_bytes, sample_rows, full_rows, torch_what, torch_bytes=None):
        def rec(kind, n_cores, dt, reps, nbytes, what):
            out.append({"config": config, "case": case, "value": round(nbytes / dt / 1e9, 3), "unit": "GB/s",
                        "us": round(dt * 1e6, 1), "cores": n_cores, "kind": kind,
                        "sample": "%d of %d rows, %s, %d repetitions, mean" % (sample_rows, full_rows, what, reps)})
        # the team size is set through the operator library itself: whichever OpenMP runtime it is bound to in this
        # process (torch ships one of its own) is the one that counts
        assert ops.set_host_threads(cores) == cores
        dt, reps = _timed_cpu(port_fn, budget_s)
        rec("port", cores, dt, reps, algo_bytes, "fp32 arithmetic")
        assert ops.set_host_threads(1) == 1
        dt, reps = _timed_cpu(port_fn, budget_s)
        rec("port (1 thread)", 1, dt, reps, algo_bytes, "fp32 arithmetic")
        ops.set_host_threads(cores)
        if torch_fn is not None:
            with torch.no_grad():
                dt, reps = _timed_cpu(torch_fn, budget_s)
            rec("torch-cpu (oneDNN-class)", cores, dt, reps, torch_bytes or algo_bytes, torch_what)

    # C1: the whole configuration, fp32 storage
    rows, cols = 8192, 4096
    x = block(rows, cols, torch.float32); y = torch.empty_like(x)
    gm, bt = torch.ones(cols), torch.zeros(cols)
    mean, var = torch.empty(rows, 1), torch.empty(rows, 1)
    add("C1", "layernorm fwd fp32 [8192x4096] (LayerNormCpu)",
        lambda: ops.layer_norm(x, gm, bt, mean, var, y, 1, 1e-5),
        lambda: torch.ops.aten.native_layer_norm(x, [cols], gm, bt, 1e-5),
        rows * (2 * cols * 4 + 8), rows, 8192, "torch native_layer_norm")
    # C5 layer norm at 5120 columns, forward and gradient, 3/4 of the rows, bf16 storage
    rows, cols = 12288, 5120
    x5 = block(rows, cols, bf); y5 = torch.empty_like(x5); dy5 = block(rows, cols, bf); dx5 = torch.empty_like(x5)
    gm5, bt5 = torch.ones(cols, dtype=bf), torch.zeros(cols, dtype=bf)
    mean5, var5 = torch.empty(rows, 1, dtype=bf), torch.empty(rows, 1, dtype=bf)
    dgm, dbt = torch.empty(cols, dtype=bf), torch.empty(cols, dtype=bf)
    _, tmean, trstd = torch.ops.aten.native_layer_norm(x5, [cols], gm5, bt5, 1e-5)
    add("C5", "layernorm fwd bf16 [16384x5120] (LayerNormCpu)",
        lambda: ops.layer_norm(x5, gm5, bt5, mean5, var5, y5, 1, 1e-5),
        lambda: torch.ops.aten.native_layer_norm(x5, [cols], gm5, bt5, 1e-5),
        rows * (2 * cols * 2 + 8), rows, 16384, "torch native_layer_norm")
    add("C5", "layernorm bwd bf16 [16384x5120] (LayerNormGradientCpu)",
        lambda: ops.layer_norm_gradient(dy5, x5, gm5, dx5, dgm, dbt, mean5, var5, 1, 1e-5),
        lambda: torch.ops.aten.native_layer_norm_backward(dy5, x5, [cols], tmean, trstd, gm5, bt5, [True, True, True]),
        rows * (3 * cols * 2 + 8), rows, 16384, "torch native_layer_norm_backward")
    # C2: 1/8 of the rows
    rows, cols = 32768, 2048
    x2 = block(rows, cols, bf); y2 = torch.empty_like(x2); dx2 = torch.empty_like(x2)
    add("C2", "softmax fwd bf16 [4,32,2048,2048] (SoftmaxCpu)", lambda: ops.softmax(x2, y2, 1),
        lambda: torch.softmax(x2, -1), 2 * rows * cols * 2, rows, 262144, "torch.softmax")
    add("C2", "softmax bwd bf16 [4,32,2048,2048] (SoftmaxGradientCpu)", lambda: ops.softmax_gradient(y2, x2, dx2, 1),
        lambda: torch.ops.aten._softmax_backward_data(x2, y2, -1, bf), 3 * rows * cols * 2, rows, 262144,
        "torch _softmax_backward_data")
    # C3: half of the rows
    rows, cols = 16384, 4096
    x3 = block(rows, cols, bf); o0 = torch.empty(cols, dtype=bf); o1 = torch.empty(rows, dtype=bf)
    for name, axes, o in (("axis 1", [1], o1), ("axis 0", [0], o0)):
        for red in ("sum", "mean"):
            tfn = (lambda a=axes[0]: torch.sum(x3, a)) if red == "sum" else (lambda a=axes[0]: torch.mean(x3, a))
            add("C3", "reduce %s %s bf16 [32768x4096] (ReduceCpu)%s" % (
                red, name, "; also the merged axes (0,1) of [64x512x4096]" if (axes == [0] and red == "sum") else ""),
                (lambda axes=axes, o=o, red=red: ops.reduce(x3, o, axes, red)), tfn, rows * cols * 2, rows, 32768,
                "torch.%s" % red)
    # C5 cross-entropy: 1/8 of the rows
    rows, cols = 2048, 32000
    xc = block(rows, cols, bf); loss = torch.empty(rows, dtype=bf); dxc = torch.empty_like(xc)
    gl = torch.full((rows,), 1.0 / 16384, dtype=bf)
    lab = (torch.arange(rows, dtype=torch.int64) * 31) % cols
    lab[::20] = IGNORE
    add("C5", "cross-entropy fwd bf16 [16384x32000] (SoftmaxCrossEntropySparseCpu)",
        lambda: ops.softmax_cross_entropy_sparse(xc, lab, loss, IGNORE),
        lambda: F.cross_entropy(xc, lab, ignore_index=IGNORE, reduction="none"),
        rows * (cols * 2 + 10), rows, 16384, "torch F.cross_entropy")
    xg = xc.clone().requires_grad_(True)

    def torch_ce_fwd_bwd():
        with torch.enable_grad():
            xg.grad = None
            F.cross_entropy(xg, lab, ignore_index=IGNORE, reduction="sum").backward()

    add("C5", "cross-entropy bwd bf16 [16384x32000] (SoftmaxCrossEntropySparseGradientCpu)",
        lambda: ops.softmax_cross_entropy_sparse_gradient(xc, lab, gl, dxc, IGNORE), torch_ce_fwd_bwd,
        rows * (2 * cols * 2 + 10), rows, 16384,
        "torch F.cross_entropy forward + autograd backward (bytes of forward and backward counted)",
        torch_bytes=rows * (3 * cols * 2 + 20))
    return out


def stream_sweep(hk, torch, steps=40):
    """The streaming roof of every read : write mix the kernels have: hipMemcpyAsync device to device, then a kernel
    that only moves 256 MiB arrays in every launch shape (workgroup size, vectors in flight per thread, non-temporal
    hints, one-shot grid or a fixed number of workgroups per compute unit).  Prints the table and returns the best
    shape per mix."""
    n = 256 << 20
    bufs = [torch.empty(n, dtype=torch.uint8, device="cuda").fill_(i + 1) for i in range(8)]

    def timed(fn):
        for i in range(10):
            fn(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    preroll(torch, lambda i: hk.memcpy_d2d(bufs[(2 * i) % 8], bufs[(2 * i + 1) % 8]))
    d = timed(lambda i: hk.memcpy_d2d(bufs[(2 * i) % 8], bufs[(2 * i + 1) % 8]))
    res = {"hipMemcpyAsync device-to-device 256 MiB": {"us": round(d * 1e6, 2), "GBps": round(2 * n / d / 1e9, 1),
                                                      "frac": round(2 * n / d / 1e9 / HBM_PEAK_GBS, 4)}}
    print("stream %-8s %-58s %8.2f us %7.1f GB/s %5.1f%%" % ("1R:1W", "hipMemcpyAsync device-to-device", d * 1e6,
                                                           2 * n / d / 1e9, 2 * n / d / 1e9 / HBM_PEAK_GBS * 100), file=sys.stderr, flush=True)
    shapes = [(bs, u, ntl, nts, 0) for bs in (64, 128, 256, 512, 1024) for u in (1, 2, 4)
              for ntl in (0, 1) for nts in (0, 1)]
    shapes += [(bs, u, 1, 1, w) for bs in (256, 512, 1024) for u in (1, 2, 4) for w in (1, 2, 4, 8)]
    for nr, nw in ((1, 1), (2, 1), (1, 2), (1, 0), (0, 1)):
        best = None
        for bs, u, ntl, nts, w in shapes:
            if (nr == 0 and ntl) or (nw == 0 and nts):
                continue

            def fn(i, bs=bs, u=u, ntl=ntl, nts=nts, w=w):
                o = (4 * i) % 8
                hk.stream_probe([bufs[(o + 2 + k) % 8] for k in range(nw)], [bufs[(o + k) % 8] for k in range(nr)],
                                bs, u, bool(ntl), bool(nts), w)
            d = timed(fn)
            gbs = (nr + nw) * n / d / 1e9
            name = "%4d threads x %d vectors, nt loads %d stores %d, %s" % (
                bs, u, ntl, nts, "one-shot grid" if w == 0 else "%d workgroups per CU" % w)
            print("stream %-8s %-58s %8.2f us %7.1f GB/s %5.1f%%" % ("%dR:%dW" % (nr, nw), name, d * 1e6, gbs,
                                                                   gbs / HBM_PEAK_GBS * 100), file=sys.stderr, flush=True)
            if best is None or gbs > best[0]:
                best = (gbs, name, d)
        res["%dR:%dW" % (nr, nw)] = {"best_shape": best[1], "us": round(best[2] * 1e6, 2), "GBps": round(best[0], 1),
                                     "frac": round(best[0] / HBM_PEAK_GBS, 4)}
    # the persistent 2R:1W walk with a ring of tiles in flight per thread and a barrier per tile: the design of the
    # backward norm kernels with the arithmetic taken out
    best = None
    for bs in (256, 512, 1024):
        for w in (1, 2):
            for depth in (1, 2, 3, 4):
                for barrier in (0, 1):
                    def fn(i, bs=bs, w=w, depth=depth, barrier=barrier):
                        o = (3 * i) % 8
                        hk.ring_probe(bufs[(o + 2) % 8], bufs[o], bufs[(o + 1) % 8], bs, depth, bool(barrier), w)
                    d = timed(fn)
                    gbs = 3 * n / d / 1e9
                    name = "%4d threads, ring depth %d, barrier %d, %d workgroups per CU" % (bs, depth, barrier, w)
                    print("ring   %-8s %-58s %8.2f us %7.1f GB/s %5.1f%%" % ("2R:1W", name, d * 1e6, gbs,
                                                                           gbs / HBM_PEAK_GBS * 100), file=sys.stderr, flush=True)
                    if barrier and (best is None or gbs > best[0]):
                        best = (gbs, name, d)
    res["2R:1W pipelined persistent, barrier per tile"] = {"best_shape": best[1], "us": round(best[2] * 1e6, 2),
                                                           "GBps": round(best[0], 1),
                                                           "frac": round(best[0] / HBM_PEAK_GBS, 4)}
    del bufs
    torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100,
                    help="untimed steps after the fixed pre-roll that every case gets")
    ap.add_argument("--all", action="store_true",
                    help="also time the kernels beyond the configurations, the yardsticks and torch's operators")
    ap.add_argument("--only", default="", help="substring filter for the kernels table (comma-separated: any of them)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel table (headline only)")
    ap.add_argument("--kernels-only", action="store_true",
                    help="only the per-kernel table (with --only: only those cases run at all, e.g. under a counter pass)")
    ap.add_argument("--kernel-steps", type=int, default=KERNEL_STEPS, help="timed launches per kernels-table entry")
    ap.add_argument("--nsets", type=int, default=3, help="rotating buffer sets (working set > cache)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); no multi-GPU path exists", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    hk = _load()
    torch.cuda.set_device(0)

    if not args.kernels_only:
        # headline: fwd + bwd at the Llama-7B token shape, exactly --steps steps after pre-roll and --warmup
        step, step_bytes, rows = case_rmsnorm(hk, torch, args.nsets, "both")
        ms, _, pre = time_case(hk, torch, step, args.steps, args.warmup, profile_main=False)
        bwd, bwd_bytes, _ = case_rmsnorm(hk, torch, args.nsets, "bwd")
        _, bwd_us, _ = time_case(hk, torch, bwd, max(args.steps, KERNEL_STEPS), args.warmup, profile_main=True)
        del step, bwd
        torch.cuda.empty_cache()

    kernels = []
    for name, make in CASES:
        if args.no_kernels or not (args.all or is_config_case(name)):
            continue
        if args.only and not any(part in name for part in args.only.split(",")):
            continue
        launch, nbytes, nrows = make(hk, torch, args.nsets)
        kms, main_us, _ = time_case(hk, torch, launch, args.kernel_steps, 0,
                                    profile_main=not getattr(launch, "no_hook", False))
        if main_us is None:
            main_us = kms * 1000
        rec = {"case": name, "us": round(kms * 1000, 2), "main_kernel_us": round(main_us, 2),
               "GBps": round(nbytes / kms / 1e6, 1), "frac": round(nbytes / kms / 1e6 / HBM_PEAK_GBS, 4),
               "main_kernel_frac": round(getattr(launch, "main_bytes", nbytes) / main_us / 1e3 / HBM_PEAK_GBS, 4),
               "rows_per_s": round(nrows / kms * 1e3), "bytes": nbytes}
        if hasattr(launch, "bytes_moved"):
            # the algorithmic bytes count every row; this kernel skips the reads of ignored rows, so the rate at
            # which bytes really moved is frac * bytes_moved_frac
            rec["bytes_moved"] = launch.bytes_moved
            rec["bytes_moved_frac"] = round(launch.bytes_moved / nbytes, 4)
            rec["ignored_rows"] = launch.ignored_rows
            rec["frac_of_bytes_moved"] = round(launch.bytes_moved / kms / 1e6 / HBM_PEAK_GBS, 4)
        kernels.append(rec)
        print("%-46s %9.2f us (main %8.2f us) %8.1f GB/s  %5.1f%% (main %5.1f%%)" % (
            name, rec["us"], rec["main_kernel_us"], rec["GBps"], 100 * rec["frac"],
            100 * rec["main_kernel_frac"]), file=sys.stderr, flush=True)
        del launch
        torch.cuda.empty_cache()

    if args.kernels_only:
        print(json.dumps({"kernel_steps": args.kernel_steps, "kernels": kernels}), flush=True)
        return
    achieved = bwd_bytes / bwd_us / 1e3
    out = {
        "metric": "HBM GB/s, RMSNorm fwd+bwd at Llama-7B token shape (algorithmic bytes / step time)",
        "value": round(step_bytes / ms / 1e6, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "preroll_steps": pre, "ms_per_step": round(ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "C4 RMSNorm fwd+bwd bf16 [32768 packed tokens x 4096], eps 1e-6, weight U(0.8,1.2)",
                   "rows": rows, "hidden": 4096, "storage": "bf16", "accumulate": "fp32", "us_fwd_plus_bwd": round(ms * 1000, 2),
                   "rows_per_s": round(rows / ms * 1e3), "frac_of_hbm_peak": round(step_bytes / ms / 1e6 / HBM_PEAK_GBS, 4)},
        "roofline": {"bound": "hbm", "kernel": "norm_bwd_kernel<bf16> (RMSNorm backward, dx + dgamma partials)",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": NORM_BWD_TRAFFIC_BYTES,
                     "algorithmic_bytes_per_launch": bwd_bytes, "avg_launch_us": round(bwd_us, 2)},
    }
    if args.all and not args.only:
        out["stream_roof"] = stream_sweep(hk, torch)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    if kernels:
        out["kernel_steps"] = args.kernel_steps
        out["kernels"] = kernels
    if not args.no_cpu and not args.no_kernels:
        out["cpu_baselines"] = cpu_baselines()
        for rec in out["cpu_baselines"]:
            print("cpu  %-3s %-66s %-26s %10.1f us %8.2f GB/s (%d threads)" % (
                rec["config"], rec["case"][:66], rec["kind"], rec["us"], rec["value"], rec["cores"]), file=sys.stderr,
                flush=True)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
