"""The committed fixtures (tests/golden/hotpath_golden.npz, written by make_golden.py) against
the CPU oracle here, and against the GPU launchers under -m gpu."""
import os

import numpy as np
import pytest

import oracle_lib as O

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hotpath_golden.npz"))


def test_oracle_reproduces_the_fixtures():
    g = GOLD
    assert np.array_equal(O.addition(g["ew_a"], g["ew_b"]), g["ew_add"])
    assert np.array_equal(O.hadamard(g["ew_a"], g["ew_b"]), g["ew_mul"])
    np.testing.assert_allclose(O.selu(g["ew_a"]), g["ew_selu"], rtol=1e-15)
    np.testing.assert_allclose(O.selu_reverse(g["ew_a"], g["ew_de"]), g["ew_selu_rev"], rtol=1e-15)
    np.testing.assert_allclose(O.fused_selu_hadamard_add_add(g["ew_a"], g["ew_b"], g["ew_c"], g["ew_d"]),
                               g["ew_e"], rtol=1e-15)
    da, db, dc, dd = O.fused_selu_hadamard_add_add_reverse(g["ew_a"], g["ew_b"], g["ew_c"], g["ew_d"], g["ew_de"])
    np.testing.assert_allclose(da, g["ew_da"], rtol=1e-15)
    np.testing.assert_allclose(dc, g["ew_dc"], rtol=1e-15)
    np.testing.assert_allclose(O.softmax_ij_j(g["sm_x"]), g["sm_y"], rtol=1e-15)
    np.testing.assert_allclose(O.softmax_ij_j_reverse(g["sm_y32"], g["sm_dy"]), g["sm_dx"], rtol=1e-14, atol=1e-18)
    np.testing.assert_allclose(O.softmax_ij_j(g["smc_x"]), g["smc_y"], rtol=1e-15)
    eps = float(g["rn_eps"])
    np.testing.assert_allclose(O.rmsnorm_ij_j(g["rn_x"], g["rn_g"], eps), g["rn_y"], rtol=1e-15)
    dx, dg = O.rmsnorm_ij_j_reverse(g["rn_x"], g["rn_g"], g["rn_dy"], eps)
    np.testing.assert_allclose(dx, g["rn_dx"], rtol=1e-14, atol=1e-18)
    np.testing.assert_allclose(dg, g["rn_dg"], rtol=1e-14, atol=1e-18)


@pytest.mark.gpu
def test_gpu_launchers_reproduce_the_fixtures():
    import torch
    import gpu_lib as G

    g = GOLD
    f32, f16 = torch.float32, torch.float16
    a, b, c, d, de = (G.dev(g[k], f32) for k in ("ew_a", "ew_b", "ew_c", "ew_d", "ew_de"))
    out = G.Guarded(a.t.shape, f32)
    G.say("golden: elementwise")
    G.addition(a.t, b.t, out.t)
    G.compare(out.t, g["ew_add"], f32, "golden add", rowwise=False)
    G.hadamard(a.t, b.t, out.t)
    G.compare(out.t, g["ew_mul"], f32, "golden hadamard", rowwise=False)
    G.selu(a.t, out.t)
    G.compare(out.t, g["ew_selu"], f32, "golden selu", rowwise=False)
    acc = G.dev(np.zeros_like(g["ew_a"]), f32)
    G.selu_reverse(a.t, acc.t, de.t)
    G.compare(acc.t, g["ew_selu_rev"], f32, "golden selu_reverse", rowwise=False)
    G.fused(a.t, b.t, c.t, d.t, out.t)
    G.compare(out.t, g["ew_e"], f32, "golden fused", rowwise=False)
    grads = [G.Guarded(a.t.shape, f32) for _ in range(4)]
    G.fused_reverse(a.t, b.t, c.t, d.t, de.t, *[x.t for x in grads])
    G.compare(grads[0].t, g["ew_da"], f32, "golden fused da", rowwise=False)
    G.compare(grads[1].t, g["ew_da"], f32, "golden fused db", rowwise=False)
    G.compare(grads[2].t, g["ew_dc"], f32, "golden fused dc", rowwise=False)
    G.compare(grads[3].t, g["ew_dc"], f32, "golden fused dd", rowwise=False)

    G.say("golden: softmax")
    x, dy, y32 = G.dev(g["sm_x"], f32), G.dev(g["sm_dy"], f32), G.dev(g["sm_y32"], f32)
    y = G.Guarded(x.t.shape, f32)
    G.softmax(x.t, y.t)
    G.compare(y.t, g["sm_y"], f32, "golden softmax", atol=1e-6)
    dx = G.Guarded(x.t.shape, f32)
    G.softmax_reverse(y32.t, dy.t, dx.t)
    G.compare(dx.t, g["sm_dx"], f32, "golden softmax reverse",
              scale=G.softmax_reverse_scale(g["sm_y32"], g["sm_dy"]))
    xm = G.dev(g["smc_x"], f16)
    ym = G.Guarded(xm.t.shape, f16)
    G.softmax(xm.t, ym.t)
    G.compare(ym.t, g["smc_y"], f16, "golden causal softmax r16", **G.softmax_tol(f16))
    assert bool((ym.t[torch.isinf(xm.t)] == 0).all())

    G.say("golden: rmsnorm")
    eps = float(g["rn_eps"])
    x, gg, dy = G.dev(g["rn_x"], f32), G.dev(g["rn_g"], f32), G.dev(g["rn_dy"], f32)
    m, n = x.t.shape
    y, dx, dg = G.Guarded((m, n), f32), G.Guarded((m, n), f32), G.Guarded((n,), f32)
    G.rmsnorm(x.t, gg.t, y.t, eps)
    G.compare(y.t, g["rn_y"], f32, "golden rmsnorm")
    scratch, _ = G.rmsnorm_scratch(f32, m, n)
    G.rmsnorm_reverse(x.t, gg.t, dy.t, dx.t, dg.t, scratch.t, eps)
    sdx, sdg = G.rmsnorm_reverse_scales(g["rn_x"], g["rn_g"], g["rn_dy"], eps)
    G.compare(dx.t, g["rn_dx"], f32, "golden rmsnorm dx", scale=sdx)
    G.compare(dg.t, g["rn_dg"], f32, "golden rmsnorm dg", rowwise=False, scale=sdg)
