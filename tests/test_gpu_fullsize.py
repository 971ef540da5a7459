"""The benchmark configurations at their full sizes: size-independent properties over the
whole output (computed on the GPU with torch reductions, which are not the code under test)
plus the fp64 oracle on a sample of rows / a slice of elements."""
import numpy as np
import pytest
import torch

import gpu_lib as G
import oracle_lib as O
from metaphor_amd import workloads as W

pytestmark = pytest.mark.gpu


def _sample_rows(m, k, seed):
    r = np.random.default_rng(seed)
    rows = np.unique(np.concatenate([[0, 1, m // 2, m - 2, m - 1], r.integers(0, m, k)]))
    return torch.from_numpy(rows).cuda()


def test_cfg1_softmax_forward_r32():
    w = W.Cfg1(seed=0)
    G.say("cfg1 softmax fwd [256,1024] r32")
    w.forward()
    torch.cuda.synchronize()
    G.compare(w.y, O.softmax_ij_j(G.host(w.x)), torch.float32, "cfg1", atol=1e-6)


def test_cfg2_rmsnorm_forward_reverse_r32():
    w = W.Cfg2(seed=0)
    G.say("cfg2 rmsnorm fwd+rev [8192,4096] r32")
    w.forward()
    w.reverse()
    torch.cuda.synchronize()
    m, n = w.shape
    # property: y / gain has mean square 1/(1 + eps/ms) ~ 1 in every row
    ms = (w.y.double() / w.gain.double()).pow(2).mean(dim=1)
    assert float((ms - 1).abs().max()) < 1e-4
    # the whole problem against the oracle (dg couples all rows)
    x, g, dy = G.host(w.x), G.host(w.gain), G.host(w.dy)
    y = O.rmsnorm_ij_j(x, g, w.eps)
    dx, dg = O.rmsnorm_ij_j_reverse_mt(x, g, dy, w.eps)
    sdx, sdg = G.rmsnorm_reverse_scales(x, g, dy, w.eps)
    G.compare(w.y, y, torch.float32, "cfg2 y")
    G.compare(w.dx, dx, torch.float32, "cfg2 dx", scale=sdx)
    G.compare(w.dgain, dg, torch.float32, "cfg2 dgain", rowwise=False, scale=sdg)


def test_cfg3_causal_softmax_forward_reverse_r16():
    w = W.Cfg3(seed=0)
    m, n = w.shape
    G.say("cfg3 softmax fwd+rev [524288,2048] r16")
    w.forward()
    w.reverse()
    torch.cuda.synchronize()
    step = 1 << 15
    for lo in range(0, m, step):
        y = w.y[lo:lo + step]
        x = w.x[lo:lo + step]
        # masked entries are exactly zero, rows sum to 1 within r16 rounding of 2048 terms
        assert bool((y[torch.isinf(x)] == 0).all())
        s = y.float().sum(dim=1)
        assert float((s - 1).abs().max()) < 4e-3
        # dx sums to ~0 along each row and vanishes where y does
        dx = w.dx[lo:lo + step]
        assert bool((dx[y == 0] == 0).all())
        assert float(dx.float().sum(dim=1).abs().max()) < 2e-2
    rows = _sample_rows(m, 96, 3)
    xs, ys, dys = G.host(w.x[rows]), G.host(w.y[rows]), G.host(w.dy[rows])
    G.compare(w.y[rows], O.softmax_ij_j(xs), torch.float16, "cfg3 y rows", **G.softmax_tol(torch.float16))
    G.compare(w.dx[rows], O.softmax_ij_j_reverse(ys, dys), torch.float16, "cfg3 dx rows",
              scale=G.softmax_reverse_scale(ys, dys))
    # first row of every (batch, head) block keeps a single entry
    firsts = torch.arange(0, m, w.block, device="cuda")
    assert bool((w.y[firsts, 0] == 1).all())


def test_cfg4_fused_chain_forward_reverse_r32():
    w = W.Cfg4(seed=0)
    G.say("cfg4 fused chain fwd+rev 2^28 r32")
    w.forward()
    w.reverse()
    torch.cuda.synchronize()
    # symmetry of the gradients, bit for bit, over the whole range
    assert torch.equal(w.da, w.db) and torch.equal(w.dc, w.dd)
    # selu's range: e > -scale*alpha everywhere
    assert float(w.e.min()) > -1.0507010 * 1.6732632 - 1e-6
    n = w.n
    for lo in (0, n // 3 + 1, n - (1 << 20)):
        sl = slice(lo, lo + (1 << 20))
        ins = [G.host(t[sl]) for t in (w.a, w.b, w.c, w.d)]
        de = G.host(w.de[sl])
        G.compare(w.e[sl], O.fused_selu_hadamard_add_add(*ins), torch.float32, f"cfg4 e @{lo}", rowwise=False)
        refs = O.fused_selu_hadamard_add_add_reverse(*ins, de)
        for name, got, ref in zip("abcd", (w.da, w.db, w.dc, w.dd), refs):
            G.compare(got[sl], ref, torch.float32, f"cfg4 d{name} @{lo}", rowwise=False)


@pytest.mark.parametrize("cls", [W.Cfg5a, W.Cfg5b], ids=["cfg5a", "cfg5b"])
def test_cfg5_vocabulary_softmax_forward_r32(cls):
    w = cls(seed=0)
    m, n = w.shape
    G.say(f"{w.name} vocabulary softmax fwd [{m},{n}] r32")
    w.forward()
    torch.cuda.synchronize()
    s = w.y.double().sum(dim=1)
    assert float((s - 1).abs().max()) < 1e-5
    # softmax preserves the order of the logits: the arg max survives
    assert torch.equal(w.y.argmax(dim=1), w.x.argmax(dim=1))
    rows = _sample_rows(m, 24, 5)
    G.compare(w.y[rows], O.softmax_ij_j(G.host(w.x[rows])), torch.float32, f"{w.name} rows", atol=1e-6)
