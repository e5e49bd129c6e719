"""Where the reference's own bf16 kernels sit: numpy emulation of the ROUNDING STEPS of three reference
GPU kernels when spec_t = bfloat16 (they do their arithmetic in the storage type).  Test infrastructure
only, informational: it shows how far the reference's results are from the exact value, so that a
comparison "ours vs. the reference within 1e-2" can be made without running the reference.

Every intermediate that the reference holds in a bfloat16 variable is rounded to bfloat16 here
(round-to-nearest-even, hetu/core/bfloat16.h:41-53); float intermediates stay float32.  The order of
additions follows the kernels' thread layout; a different GPU would reorder nothing, the layout is fixed
by the launch shape.

  softmax_fwd      hetu/impl/kernel/Softmax.cu:199-248 (softmax_kernel2), launch :262-308
  sce_sparse_fwd   hetu/impl/kernel/SoftmaxCrossEntropySparse.cu:11-55
  layernorm_fwd    hetu/impl/kernel/LayerNorm.cu:15-64, launch :86-88
  block reductions hetu/impl/utils/cuda_math.h:596-613 (warp shuffle tree, then one warp over the warp sums)
"""
import numpy as np

from . import round_bf16

F32 = np.float32


def _rb(a):
    return round_bf16(np.asarray(a, dtype=F32))


def _tree_sum(v, rnd):
    """shfl_down tree over the last axis (a power of two): lane 0 ends with the total."""
    v = v.copy()
    k = v.shape[-1] // 2
    while k >= 1:
        v[..., :k] = rnd(v[..., :k] + v[..., k:2 * k])
        k //= 2
    return v[..., 0]


def _block_sum(per_thread, rnd, warp=32):
    """BlockReduceSum: warp trees, then warp 0 sums the per-warp results (missing warps count as zero)."""
    rows, threads = per_thread.shape
    nwarps = (threads + warp - 1) // warp
    padded = np.zeros((rows, nwarps * warp), dtype=F32)
    padded[:, :threads] = per_thread
    warp_sums = _tree_sum(padded.reshape(rows, nwarps, warp), rnd)
    lanes = np.zeros((rows, warp), dtype=F32)
    lanes[:, :nwarps] = warp_sums
    return _tree_sum(lanes, rnd)


def softmax_fwd(x, threads_per_row=64, bf16=True):
    """x: [rows, cols] float32 holding bf16 values.  Per thread a contiguous chunk of
    ceil(cols / threads) elements; maximum exact; exp(x - max) and the running sum in spec_t;
    out = exp(x - max) / sum in spec_t."""
    rnd = _rb if bf16 else (lambda a: np.asarray(a, dtype=F32))
    x = np.asarray(x, dtype=F32)
    rows, cols = x.shape
    per = (cols + threads_per_row - 1) // threads_per_row
    used = (cols + per - 1) // per
    m = x.max(axis=1, keepdims=True)
    e = rnd(np.exp(rnd(x - m).astype(np.float64)))           # hexp(bf16): exp, rounded to the type
    pad = np.zeros((rows, used * per), dtype=F32)
    pad[:, :cols] = e
    chunks = pad.reshape(rows, used, per)
    acc = np.zeros((rows, used), dtype=F32)
    for j in range(per):                                       # sum_thread += ..., rounded at every step
        acc = rnd(acc + chunks[:, :, j])
    p2 = 1
    while p2 < used:
        p2 *= 2
    lanes = np.zeros((rows, p2), dtype=F32)
    lanes[:, :used] = acc
    total = _tree_sum(lanes, rnd)[:, None]
    return rnd(e / total)


def sce_sparse_fwd(x, labels, ignored_index, threads=1024, bf16=True):
    """loss = -x[label] + max + spec_t(log(sum)); (x - max) is rounded to spec_t before the float exp,
    the sum is float32 (strided per-thread sums, block tree)."""
    rnd = _rb if bf16 else (lambda a: np.asarray(a, dtype=F32))
    x = np.asarray(x, dtype=F32)
    rows, cols = x.shape
    threads = min(max(32, cols), threads)
    m = x.max(axis=1, keepdims=True)
    e = np.exp(rnd(x - m).astype(F32)).astype(F32)             # expf(float(spec_t difference))
    per = (cols + threads - 1) // threads
    pad = np.zeros((rows, per * threads), dtype=F32)
    pad[:, :cols] = e
    strided = pad.reshape(rows, per, threads)                  # thread t takes t, t + threads, ...
    acc = np.zeros((rows, threads), dtype=F32)
    for j in range(per):
        acc = (acc + strided[:, j, :]).astype(F32)
    total = _block_sum(acc, lambda a: np.asarray(a, dtype=F32))
    lab = np.asarray(labels, dtype=np.int64)
    valid = lab != ignored_index
    xl = x[np.arange(rows), np.where(valid, lab, 0)]
    t1 = rnd(-xl + m[:, 0])
    loss = rnd(t1 + rnd(np.log(total).astype(F32)))
    return np.where(valid, loss, F32(0)).astype(F32)


def layernorm_fwd(x, gamma, beta, eps, bf16=True):
    """Sum and sum of squares accumulate in spec_t (strided per thread, block tree);
    var = E[x^2] - mean^2 clamped at 0, all in spec_t; y = (x - mean) * rsqrt * gamma + beta in spec_t."""
    rnd = _rb if bf16 else (lambda a: np.asarray(a, dtype=F32))
    x = np.asarray(x, dtype=F32)
    rows, cols = x.shape
    threads = 1024 if cols >= 1024 else 64
    per = (cols + threads - 1) // threads
    pad = np.zeros((rows, per * threads), dtype=F32)
    pad[:, :cols] = x
    strided = pad.reshape(rows, per, threads)
    s = np.zeros((rows, threads), dtype=F32)
    q = np.zeros((rows, threads), dtype=F32)
    for j in range(per):
        s = rnd(s + strided[:, j, :])
        q = rnd(q + rnd(strided[:, j, :] * strided[:, j, :]))
    mean = rnd(_block_sum(s, rnd) / F32(cols))
    var = rnd(rnd(_block_sum(q, rnd) / F32(cols)) - rnd(mean * mean))
    var = np.where(var < 0, F32(0), var)
    tmp = rnd(F32(1.0) / np.sqrt(var.astype(F32) + F32(eps)))
    y = rnd(rnd(rnd(rnd(x - mean[:, None]) * tmp[:, None]) * np.asarray(gamma, dtype=F32)[None, :])
            + np.asarray(beta, dtype=F32)[None, :])
    return y, mean, var
