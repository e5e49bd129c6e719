"""Shared helpers of the test-suite: package loading, synthetic inputs of the
benchmark configurations, dtype plumbing and the comparison rule."""
import importlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import oracle  # noqa: E402  (test infrastructure)

# Tolerances of the parity bar: fp32 within 1e-5 relative, bf16 / fp16 within
# 1e-2 relative (fp32 accumulation).  "Relative" is taken against
# |expected| + rms(expected): elements that cancel to ~0 are judged against the
# tensor's scale instead of their own vanishing magnitude.
RTOL = {"fp32": 1e-5, "bf16": 1e-2, "fp16": 1e-2, "fp64": 1e-12}


def load_package():
    return importlib.import_module("hotspa-ae_amd")


def to_torch(a, dtype, device):
    """numpy array (values already representable in `dtype`) -> torch tensor."""
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype in ("fp32", "bf16", "fp16", "fp64"):
        td = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16, "fp64": torch.float64}[dtype]
        t = t.to(td)
    return t.to(device)


def to_numpy(t):
    import torch
    if t.dtype in (torch.bfloat16, torch.float16):
        t = t.float()
    return t.detach().cpu().numpy()


def rel_error(actual, expected, scale=None):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    if scale is None:
        scale = float(np.sqrt(np.mean(np.square(expected)))) if expected.size else 0.0
    denom = np.abs(expected) + scale
    denom = np.where(denom == 0.0, 1.0, denom)
    return np.abs(actual - expected) / denom


def assert_close(actual, expected, dtype, what="", scale=None, rtol=None):
    """actual: torch tensor or numpy; expected: float64 numpy (oracle)."""
    if hasattr(actual, "detach"):
        actual = to_numpy(actual)
    actual = np.asarray(actual, dtype=np.float64).reshape(np.asarray(expected).shape)
    assert np.all(np.isfinite(actual) == np.isfinite(expected)), "%s: non-finite pattern differs" % what
    fin = np.isfinite(expected)
    err = rel_error(actual[fin], np.asarray(expected)[fin], scale)
    worst = float(err.max()) if err.size else 0.0
    tol = RTOL[dtype] if rtol is None else rtol
    assert worst <= tol, "%s: max relative error %.3e exceeds %.1e" % (what, worst, tol)
    return worst


def rng(seed):
    return np.random.default_rng(seed)


def draw(seed, shape, dist="normal", a=0.0, b=1.0, dtype="fp32"):
    """fp32 draw, then rounded to the storage dtype (returned as fp32)."""
    g = rng(seed)
    if dist == "normal":
        v = g.standard_normal(shape, dtype=np.float32) * np.float32(b) + np.float32(a)
    else:
        v = g.random(shape, dtype=np.float32) * np.float32(b - a) + np.float32(a)
    return oracle.round_to(v, dtype)


def packed_lengths(seed=401, total=32768, mu=6.5, sigma=1.0, lo=128, hi=16384):
    """Variable-length sequences packed until `total` tokens (the boundaries do
    not enter the row-wise kernels; recorded for completeness)."""
    g = rng(seed)
    lens = []
    while sum(lens) < total:
        n = int(np.clip(np.round(g.lognormal(mu, sigma)), lo, hi))
        lens.append(min(n, total - sum(lens)))
    return lens
