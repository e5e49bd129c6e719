"""CPU restatement (numpy, float64) of the full dropout-add-LayerNorm / RMSNorm interface.

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the benchmark's CPU leg; the product
path never calls it.

Follows the flash-attention layer_norm kernels vendored by the reference (third_party/flash_attn,
include/layer_norm):
  forward            ln_fwd_kernels.cuh:66-186       (dropout, rowscale, colscale, row subsets, residual)
  backward           ln_bwd_kernels.cuh:93-221       (dx0, dresidual, dgamma, dbeta, dcolscale)
  parallel forward   ln_parallel_residual_fwd_kernels.cuh:60-190
  parallel backward  ln_parallel_residual_bwd_kernels.cuh:88-185
and their launchers hetu/impl/kernel/RMSNorm.cu:91-264, 266-470, 474-826.

The dropout mask.  The reference draws curand_uniform per element from a Philox4x32-10 stream keyed by the
CUDA thread index of a persistent grid sized from the SM count, so its mask is a property of the device it
ran on, not of the inputs, and cannot be reproduced.  Here the mask is a pure function of (seed, offset,
element index): element e of x0 uses word e % 4 of philox4x32_10(counter = (2 * (e // 4) + which, offset),
key = seed) (which = 1 for the second input of the parallel form), mapped to (0, 1] exactly like
curand_uniform (u * 2^-32 + 2^-33 in float32), kept when <= 1 - p.

Pinned by: the Random123 known-answer vectors for philox4x32-10; torch.autograd on the composed function
for every gradient (tests/test_oracle_dropout_ln.py); reduction to the plain norm oracle without features.
"""
import numpy as np

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_W0 = 0x9E3779B9
_W1 = 0xBB67AE85
_MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter, key):
    """counter: uint32 [..., 4], key: uint32 [..., 2] (broadcastable) -> uint32 [..., 4].
    Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3" (SC'11), 10 rounds."""
    counter = np.asarray(counter, dtype=np.uint32)
    key = np.asarray(key, dtype=np.uint32)
    c = [counter[..., i].astype(np.uint64) for i in range(4)]
    k0 = key[..., 0].astype(np.uint64)
    k1 = key[..., 1].astype(np.uint64)
    for r in range(10):
        p0 = _M0 * c[0]
        p1 = _M1 * c[2]
        n0 = ((p1 >> np.uint64(32)) ^ c[1] ^ k0) & _MASK32
        n1 = p1 & _MASK32
        n2 = ((p0 >> np.uint64(32)) ^ c[3] ^ k1) & _MASK32
        n3 = p0 & _MASK32
        c = [n0, n1, n2, n3]
        k0 = (k0 + np.uint64(_W0)) & _MASK32
        k1 = (k1 + np.uint64(_W1)) & _MASK32
    return np.stack(c, axis=-1).astype(np.uint32)


def uniform_from_bits(bits):
    """curand_uniform's map of 32 random bits to (0, 1]: float32(bits) * 2^-32 + 2^-33, one rounding."""
    f = np.asarray(bits, dtype=np.uint32).astype(np.float32).astype(np.float64)   # round to nearest even
    return (f * 2.0 ** -32 + 2.0 ** -33).astype(np.float32)


def dropout_keep(seed, offset, numel, keep_p, which=0):
    """uint8 [numel]: 1 where element e is kept."""
    groups = (numel + 3) // 4
    g = 2 * np.arange(groups, dtype=np.uint64) + np.uint64(which)
    ctr = np.empty((groups, 4), dtype=np.uint32)
    ctr[:, 0] = (g & _MASK32).astype(np.uint32)
    ctr[:, 1] = (g >> np.uint64(32)).astype(np.uint32)
    ctr[:, 2] = np.uint32(offset & 0xFFFFFFFF)
    ctr[:, 3] = np.uint32((offset >> 32) & 0xFFFFFFFF)
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint32)
    bits = philox4x32_10(ctr, key).reshape(-1)[:numel]
    return (uniform_from_bits(bits) <= np.float32(keep_p)).astype(np.uint8)


def _f64(a):
    return None if a is None else np.asarray(a, dtype=np.float64)


def _norm_rows(x, eps, is_rms):
    mu = x.mean(axis=1)
    m2 = ((x - mu[:, None]) ** 2).sum(axis=1)
    cols = x.shape[1]
    # ln_fwd_kernels.cuh:159: rs = rsqrt(m2 / cols + eps + (is_rms ? mu^2 : 0))
    rs = 1.0 / np.sqrt(m2 / cols + eps + (mu * mu if is_rms else 0.0))
    y = rs[:, None] * (x - (0.0 if is_rms else mu[:, None]))
    return mu, rs, y


def fwd(x0, residual, gamma, beta, rowscale=None, colscale=None, x0_subset=None, z_subset=None, dmask=None,
        dropout_p=0.0, eps=1e-5, rowscale_const=1.0, z_numrows=None, is_rms=False):
    """ln_fwd_kernels.cuh:97-182.  dmask: uint8 keep mask of x0's shape (required when dropout_p > 0).
    Subsets are 1-based row numbers, 0 = "no row" (x0 contributes nothing / z is not written).
    Returns z [z_numrows or rows, cols] (rows never written stay NaN), x [rows, cols], mu, rs."""
    x0 = _f64(x0); residual = _f64(residual); gamma = _f64(gamma); beta = _f64(beta)
    rowscale = _f64(rowscale); colscale = _f64(colscale)
    cols = x0.shape[1]
    has_subset = x0_subset is not None
    rows = len(x0_subset) if has_subset else x0.shape[0]
    scale = 1.0 / (1.0 - dropout_p)
    x = np.zeros((rows, cols))
    for r in range(rows):
        rsv = rowscale_const if has_subset else (1.0 if rowscale is None else rowscale[r])
        row_x0 = int(x0_subset[r]) if has_subset else r + 1
        if row_x0 > 0:
            v = x0[row_x0 - 1] * rsv
            if dropout_p > 0.0:
                v = np.where(dmask[row_x0 - 1] != 0, v * scale, 0.0)
            if colscale is not None:
                v = v * colscale
            x[r] = v
        if residual is not None:
            x[r] = x[r] + residual[r]
    mu, rs, y = _norm_rows(x, eps, is_rms)
    zfull = y * gamma[None, :] + (0.0 if beta is None else beta[None, :])
    if has_subset:
        z = np.full((int(z_numrows), cols), np.nan)
        for r in range(rows):
            row_z = int(z_subset[r])
            if row_z > 0:
                z[row_z - 1] = zfull[r]
    else:
        z = zfull
    return z, x, mu, rs


def bwd(dz, dx_in, x, x0, dmask, mu, rs, gamma, rowscale=None, colscale=None, x0_subset=None, z_subset=None,
        dropout_p=0.0, rowscale_const=1.0, x0_numrows=None, is_rms=False):
    """ln_bwd_kernels.cuh:93-221.  Returns dx0 [x0_numrows or rows, cols] (rows never written stay NaN),
    dresidual [rows, cols], dgamma, dbeta, dcolscale (None without colscale)."""
    dz = _f64(dz); dx_in = _f64(dx_in); x = _f64(x); x0 = _f64(x0); gamma = _f64(gamma)
    mu = _f64(mu); rs = _f64(rs); rowscale = _f64(rowscale); colscale = _f64(colscale)
    rows, cols = x.shape
    has_subset = x0_subset is not None
    scale = 1.0 / (1.0 - dropout_p)
    n0 = int(x0_numrows) if has_subset else rows
    dx0 = np.full((n0, cols), np.nan)
    dres = np.zeros((rows, cols))
    dgamma = np.zeros(cols); dbeta = np.zeros(cols)
    dcol = np.zeros(cols) if colscale is not None else None
    for r in range(rows):
        rsv = rowscale_const if has_subset else (1.0 if rowscale is None else rowscale[r])
        row_z = int(z_subset[r]) if has_subset else r + 1
        row_x0 = int(x0_subset[r]) if has_subset else r + 1
        if row_z > 0:
            dzr = dz[row_z - 1]
            y = rs[r] * (x[r] - (0.0 if is_rms else mu[r]))
            dy = gamma * dzr
            mdy = 0.0 if is_rms else dy.mean()
            mdyy = (dy * y).mean()
            dxr = rs[r] * (dy - (mdyy * y + mdy))
            dgamma += dzr * y
            dbeta += dzr
        else:
            dxr = np.zeros(cols)
        if dx_in is not None:
            dxr = dxr + dx_in[r]
        dres[r] = dxr
        if row_x0 > 0:
            v = dxr * rsv
            keep = np.ones(cols, dtype=bool)
            if dropout_p > 0.0:
                v = v * scale
                keep = dmask[row_x0 - 1] != 0
            if colscale is not None:
                dcol += np.where(keep, v * x0[row_x0 - 1], 0.0)
                v = v * colscale
            dx0[row_x0 - 1] = np.where(keep, v, 0.0)
    return dx0, dres, dgamma, dbeta, dcol


def parallel_fwd(x0, x1, residual, gamma0, beta0, gamma1, beta1, dmask0=None, dmask1=None, dropout_p=0.0,
                 eps=1e-5, is_rms=False):
    """ln_parallel_residual_fwd_kernels.cuh:99-190: x = drop(x0) + drop(x1) + residual, two affine outputs
    of one normalisation.  Returns z0, z1 (None when gamma1 is None), x, mu, rs."""
    x0 = _f64(x0); x1 = _f64(x1); residual = _f64(residual)
    gamma0 = _f64(gamma0); beta0 = _f64(beta0); gamma1 = _f64(gamma1); beta1 = _f64(beta1)
    scale = 1.0 / (1.0 - dropout_p)
    x = x0.copy()
    if dropout_p > 0.0:
        x = np.where(np.asarray(dmask0) != 0, x * scale, 0.0)
    if x1 is not None:
        v = x1
        if dropout_p > 0.0:
            v = np.where(np.asarray(dmask1) != 0, v * scale, 0.0)
        x = x + v
    if residual is not None:
        x = x + residual
    mu, rs, y = _norm_rows(x, eps, is_rms)
    z0 = y * gamma0[None, :] + (0.0 if beta0 is None else beta0[None, :])
    z1 = None
    if gamma1 is not None:
        z1 = y * gamma1[None, :] + (0.0 if beta1 is None else beta1[None, :])
    return z0, z1, x, mu, rs


def parallel_bwd(dz0, dz1, dx_in, x, dmask0, dmask1, mu, rs, gamma0, gamma1, dropout_p=0.0, has_x1=True,
                 is_rms=False):
    """ln_parallel_residual_bwd_kernels.cuh:93-185.  Returns dx0, dx1 (None without x1), dresidual,
    dgamma0, dbeta0, dgamma1, dbeta1 (None when gamma1 is None)."""
    dz0 = _f64(dz0); dz1 = _f64(dz1); dx_in = _f64(dx_in); x = _f64(x)
    mu = _f64(mu); rs = _f64(rs); gamma0 = _f64(gamma0); gamma1 = _f64(gamma1)
    scale = 1.0 / (1.0 - dropout_p)
    y = rs[:, None] * (x - (0.0 if is_rms else mu[:, None]))
    dy = gamma0[None, :] * dz0
    if gamma1 is not None:
        dy = dy + gamma1[None, :] * dz1
    mdy = 0.0 if is_rms else dy.mean(axis=1, keepdims=True)
    mdyy = (dy * y).mean(axis=1, keepdims=True)
    dx = rs[:, None] * (dy - (mdyy * y + mdy))
    if dx_in is not None:
        dx = dx + dx_in
    dres = dx
    if dropout_p > 0.0:
        dx0 = np.where(np.asarray(dmask0) != 0, dx * scale, 0.0)
        dx1 = np.where(np.asarray(dmask1) != 0, dx * scale, 0.0) if has_x1 else None
    else:
        dx0 = dx
        dx1 = dx if has_x1 else None
    dg0 = (dz0 * y).sum(axis=0); db0 = dz0.sum(axis=0)
    dg1 = db1 = None
    if gamma1 is not None:
        dg1 = (dz1 * y).sum(axis=0); db1 = dz1.sum(axis=0)
    return dx0, dx1, dres, dg0, db0, dg1, db1
