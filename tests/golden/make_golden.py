#!/usr/bin/env python3
"""Writes tests/golden/rowwise_small.npz: small seeded inputs of every operator
with the float64 outputs of the CPU oracle (oracle/oracle.c).

The reference repository holds no golden vectors for these kernels and cannot
be built or imported here, so these fixtures are produced by the oracle alone;
they freeze its results so that later changes to the oracle or to the kernels
are caught.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import helpers  # noqa: E402
import oracle  # noqa: E402


def main():
    out = {}
    for dt in ("fp32", "bf16"):
        rows, cols = 6, 40
        x = helpers.draw(1, (rows, cols), dtype=dt)
        gamma = helpers.draw(2, (cols,), "uniform", 0.5, 1.5, dt)
        beta = helpers.draw(3, (cols,), "normal", 0.0, 0.1, dt)
        dy = helpers.draw(4, (rows, cols), dtype=dt)
        y, mean, var, rstd = oracle.layernorm_fwd(x, gamma, beta, 1e-5)
        dx, dg, db = oracle.layernorm_bwd(dy, x, gamma, mean.astype(np.float32), rstd.astype(np.float32), 1e-5, True)
        z, _, mu, rs = oracle.dropout_add_ln_fwd(x, None, gamma, None, 1e-6, True)
        rdx, rdg, rdb = oracle.dropout_add_ln_bwd(dy, None, x, mu.astype(np.float32), rs.astype(np.float32), gamma, True)
        sx = helpers.draw(5, (4, 3, 24), "normal", 0.0, 3.0, dt)
        sy = oracle.softmax_fwd(sx, -1)
        sdy = helpers.draw(6, (4, 3, 24), dtype=dt)
        sdx = oracle.softmax_bwd(oracle.round_to(sy, dt), sdy, -1)
        lab = np.array([3, -100, 0, 39, 17, -100], dtype=np.int64)
        loss = oracle.sce_sparse_fwd(x, lab, -100)
        gl = helpers.draw(7, (rows,), "uniform", 0.5, 1.5, dt)
        dlog = oracle.sce_sparse_bwd(x, lab, gl, -100)
        r0 = oracle.reduce(sx, [0, 1], "sum")
        r1 = oracle.reduce(sx, [2], "mean")
        for k, v in dict(x=x, gamma=gamma, beta=beta, dy=dy, ln_y=y, ln_mean=mean, ln_var=var, ln_rstd=rstd,
                         ln_dx=dx, ln_dgamma=dg, ln_dbeta=db, rms_z=z, rms_mu=mu, rms_rs=rs, rms_dx=rdx,
                         rms_dgamma=rdg, rms_dbeta=rdb, sm_x=sx, sm_y=sy, sm_dy=sdy, sm_dx=sdx, labels=lab,
                         sce_loss=loss, grad_loss=gl, sce_dlogits=dlog, red_sum01=r0, red_mean2=r1).items():
            out["%s/%s" % (dt, k)] = v
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rowwise_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
