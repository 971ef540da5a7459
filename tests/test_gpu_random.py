"""Seeded random shapes, alignments and blends through the row and matrix launchers, against the
oracle, with canaries around every buffer: the shapes no hand-written list thinks of (rows of a few
elements, rows of 200000, one-element shifts of any operand, in-place calls)."""
import numpy as np
import pytest
import torch

import gpu_lib as G
import oracle_lib as O

pytestmark = pytest.mark.gpu

DT = [torch.float32, torch.float16, torch.float64]
NAMES = ["softmax", "softmax_rev", "rmsnorm", "rmsnorm_rev", "reduce_bcast", "permutate", "inplace"]


def _shape(r):
    kind = r.integers(0, 5)
    if kind == 0:
        return int(r.integers(1, 40)), int(r.integers(1, 200))
    if kind == 1:
        return int(r.integers(1, 3000)), int(r.integers(1, 70))
    if kind == 2:
        return int(r.integers(1, 300)), int(r.integers(200, 5000))
    if kind == 3:
        return int(r.integers(1, 12)), int(r.integers(5000, 70000))
    return int(r.integers(1, 6)), int(r.integers(60000, 200000))


@pytest.mark.parametrize("seed", [11, 12])
def test_random_cases_match_the_oracle(seed):
    r = np.random.default_rng(seed)
    for case in range(150):
        dt = DT[int(r.choice([0, 0, 1, 1, 2]))]
        m, n = _shape(r)
        if dt == torch.float64 and m * n > 2_000_000:
            m = max(1, 2_000_000 // n)
        sh = [int(x) for x in r.integers(0, 2, 5)]
        alpha = float(r.choice([0.0, 0.0, 1.0, -0.5]))
        op = int(r.integers(0, 7))
        name = NAMES[op]
        G.say(f"case {case} {name} dtype={dt} m={m} n={n} shifts={sh} alpha={alpha}")
        x = G.dev(r.normal(0, 2, (m, n)), dt, sh[0])
        if op == 0:
            y = G.Guarded((m, n), dt, sh[1])
            G.softmax(x.t, y.t)
            G.compare(y.t, O.softmax_ij_j(G.host(x.t)), dt, name, **G.softmax_tol(dt))
            y.check(name)
        elif op == 1:
            y = G.Guarded((m, n), dt, sh[0])
            G.softmax(x.t, y.t)
            dy = G.dev(r.normal(0, 1, (m, n)), dt, sh[1])
            dx = G.dev(r.normal(0, 1, (m, n)), dt, sh[2])
            before = G.host(dx.t).copy()
            G.softmax_reverse(y.t, dy.t, dx.t, alpha)
            yh, dyh = G.host(y.t), G.host(dy.t)
            G.compare(dx.t, O.softmax_ij_j_reverse(yh, dyh, before if alpha else None, alpha), dt, name,
                      scale=G.softmax_reverse_scale(yh, dyh, before if alpha else None, alpha)); dx.check(name)
        elif op == 2:
            g = G.dev(r.normal(1, 0.02, n), dt, sh[1])
            y = G.Guarded((m, n), dt, sh[2])
            G.rmsnorm(x.t, g.t, y.t, 1e-6)
            G.compare(y.t, O.rmsnorm_ij_j(G.host(x.t), G.host(g.t), 1e-6), dt, name)
            y.check(name)
        elif op == 3:
            g = G.dev(r.normal(1, 0.02, n), dt, sh[1])
            dy = G.dev(r.normal(0, 1, (m, n)), dt, sh[2])
            dx = G.dev(r.normal(0, 1, (m, n)), dt, sh[3])
            dg = G.dev(r.normal(0, 1, n), dt, sh[4])
            hdx, hdg = G.host(dx.t).copy(), G.host(dg.t).copy()
            sc, _ = G.rmsnorm_scratch(dt, m, n)
            G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, sc.t, 1e-6, alpha)
            xh, gh, dyh = G.host(x.t), G.host(g.t), G.host(dy.t)
            rdx, rdg = O.rmsnorm_ij_j_reverse(xh, gh, dyh, 1e-6, hdx if alpha else None, hdg if alpha else None, alpha)
            sdx, sdg = G.rmsnorm_reverse_scales(xh, gh, dyh, 1e-6, hdx if alpha else None, hdg if alpha else None, alpha)
            G.compare(dx.t, rdx, dt, name + " dx", scale=sdx)
            G.compare(dg.t, rdg, dt, name + " dg", rowwise=False, scale=sdg)
            for b in (dx, dg, sc): b.check(name)
        elif op == 4:
            si = G.dev(r.normal(0, 1, m), dt, sh[1])
            sj = G.dev(r.normal(0, 1, n), dt, sh[2])
            bi, bj = G.host(si.t).copy(), G.host(sj.t).copy()
            xh = G.host(x.t)
            mag = np.abs(xh.astype(np.float64))
            G.matrix_op("reduce_ij_i", x.t, si.t, alpha, m, n)
            G.matrix_op("reduce_ij_j", x.t, sj.t, alpha, m, n)
            G.compare(si.t, O.reduce_ij_i(xh, bi if alpha else None, alpha), dt, "reduce_ij_i", rowwise=False, scale=mag.sum(1) + abs(alpha) * np.abs(bi.astype(np.float64)))
            G.compare(sj.t, O.reduce_ij_j(xh, bj if alpha else None, alpha), dt, "reduce_ij_j", rowwise=False, scale=mag.sum(0) + abs(alpha) * np.abs(bj.astype(np.float64)))
            d1 = G.dev(r.normal(0, 1, (m, n)), dt, sh[3])
            d2 = G.dev(r.normal(0, 1, (m, n)), dt, sh[4])
            b1, b2 = G.host(d1.t).copy(), G.host(d2.t).copy()
            G.matrix_op("broadcast_i_ij", si.t, d1.t, alpha, m, n)
            G.matrix_op("broadcast_j_ij", sj.t, d2.t, alpha, m, n)
            G.compare(d1.t, O.broadcast_i_ij(G.host(si.t), m, n, b1 if alpha else None, alpha), dt, "broadcast_i_ij", rowwise=False, scale=np.abs(b1.astype(np.float64)) * abs(alpha) + np.abs(G.host(si.t).astype(np.float64))[:, None])
            G.compare(d2.t, O.broadcast_j_ij(G.host(sj.t), m, n, b2 if alpha else None, alpha), dt, "broadcast_j_ij", rowwise=False, scale=np.abs(b2.astype(np.float64)) * abs(alpha) + np.abs(G.host(sj.t).astype(np.float64))[None, :])
            for b in (si, sj, d1, d2): b.check(name)
        elif op == 5:
            d = G.dev(r.normal(0, 1, (n, m)), dt, sh[1])
            before = G.host(d.t).copy()
            G.permutate(x.t, d.t, alpha)
            G.compare(d.t, O.permutate_ij_ji(G.host(x.t), before if alpha else None, alpha), dt, name, rowwise=False,
                      scale=np.abs(G.host(x.t).T.astype(np.float64)) + abs(alpha) * np.abs(before.astype(np.float64))); d.check(name)
        else:
            xh = G.host(x.t).copy()
            g = G.dev(r.normal(1, 0.02, n), dt, sh[1])
            if r.integers(0, 2):
                G.softmax(x.t, x.t)
                G.compare(x.t, O.softmax_ij_j(xh), dt, "softmax in place", **G.softmax_tol(dt))
            else:
                G.rmsnorm(x.t, g.t, x.t, 1e-6)
                G.compare(x.t, O.rmsnorm_ij_j(xh, G.host(g.t), 1e-6), dt, "rmsnorm in place")
        x.check(name)
