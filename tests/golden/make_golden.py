"""Writes tests/golden/hotpath_golden.npz: small seeded inputs and fp64 expected outputs for
every launcher of the hot path.

The reference ships no fixtures for this path, so these are produced by the CPU oracle
(oracle/mp_oracle.c) after tests/test_oracle.py has pinned it, and every entry is
cross-checked here against an independent fp64 library routine (torch) before it is written.
Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as O  # noqa: E402

torch.set_default_dtype(torch.float64)


def t64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64).copy())


def main():
    r = np.random.default_rng(20240607)
    out = {}

    # ---- elementwise chain, r32, n = 1000 (U(-2,2) inputs, N(0,1) upstream)
    n = 1000
    a, b, c, d = (r.uniform(-2, 2, n).astype(np.float32) for _ in range(4))
    de = r.normal(0, 1, n).astype(np.float32)
    e = O.fused_selu_hadamard_add_add(a, b, c, d)
    grads = O.fused_selu_hadamard_add_add_reverse(a, b, c, d, de)
    ts = [t64(z).requires_grad_(True) for z in (a, b, c, d)]
    te = torch.nn.functional.selu((ts[0] + ts[1]) * (ts[2] + ts[3]))
    te.backward(t64(de))
    np.testing.assert_allclose(e, te.detach().numpy(), rtol=4e-8)
    for g, t in zip(grads, ts):
        np.testing.assert_allclose(g, t.grad.numpy(), rtol=6e-8, atol=1e-300)
    out.update(ew_a=a, ew_b=b, ew_c=c, ew_d=d, ew_de=de, ew_e=e, ew_da=grads[0], ew_dc=grads[2],
               ew_add=O.addition(a, b), ew_mul=O.hadamard(a, b), ew_selu=O.selu(a),
               ew_selu_rev=O.selu_reverse(a, de))

    # ---- softmax, r32 [6, 333] and causal r16 [8, 8]
    x = (4.0 * r.normal(0, 1, (6, 333))).astype(np.float32)
    dy = r.normal(0, 1, x.shape).astype(np.float32)
    y = O.softmax_ij_j(x)
    xt = t64(x).requires_grad_(True)
    yt = torch.softmax(xt, -1)
    yt.backward(t64(dy))
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-13)
    y32 = y.astype(np.float32)
    dx = O.softmax_ij_j_reverse(y32, dy)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=0, atol=3e-7)  # y rounded to r32 first
    out.update(sm_x=x, sm_dy=dy, sm_y=y, sm_y32=y32, sm_dx=dx)

    xm = r.normal(0, 2, (8, 8))
    rows, cols = np.indices(xm.shape)
    xm[cols > rows] = -np.inf
    xm = xm.astype(np.float16)
    ym = O.softmax_ij_j(xm)
    np.testing.assert_allclose(ym, torch.softmax(t64(xm), -1).numpy(), rtol=1e-13)
    out.update(smc_x=xm, smc_y=ym)

    # ---- RMSNorm, r32 [9, 260], eps 1e-6
    m, n, eps = 9, 260, 1e-6
    x = r.normal(0, 1, (m, n)).astype(np.float32)
    g = r.normal(1, 0.02, n).astype(np.float32)
    dy = r.normal(0, 1, (m, n)).astype(np.float32)
    y = O.rmsnorm_ij_j(x, g, eps)
    dx, dg = O.rmsnorm_ij_j_reverse(x, g, dy, eps)
    xt, gt = t64(x).requires_grad_(True), t64(g).requires_grad_(True)
    yt = torch.nn.functional.rms_norm(xt, (n,), gt, eps)
    yt.backward(t64(dy))
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-13)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-10, atol=1e-14)
    np.testing.assert_allclose(dg, gt.grad.numpy(), rtol=1e-10, atol=1e-14)
    out.update(rn_x=x, rn_g=g, rn_dy=dy, rn_y=y, rn_dx=dx, rn_dg=dg, rn_eps=np.float64(eps))

    path = os.path.join(HERE, "hotpath_golden.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
