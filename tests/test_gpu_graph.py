"""The launchers under HIP graph capture: they enqueue kernels only (no allocation, no memset
nodes: the shared-row softmax clears its slots with a fill kernel), so a captured sequence can be
replayed; so can an expression fused at run time once its first call has compiled it. Every replay is checked against the eager result, with eager work and synchronisation
between replays."""
import numpy as np
import pytest
import torch

import gpu_lib as G
from metaphor_amd import workloads as W

pytestmark = pytest.mark.gpu


def test_replays_of_a_captured_forward_and_reverse_sequence_match_eager():
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    f32 = torch.float32
    m, n = 64, 4096
    # every tensor names its dtype: the session's default dtype is float64 once tests/test_oracle.py
    # has been imported, and the workspaces below are sized for r32
    rnd = lambda *shape: torch.randn(*shape, generator=gen, device="cuda", dtype=f32)
    x = rnd(m, n)
    gain = 1 + 0.02 * rnd(n)
    dy = rnd(m, n)
    y, dx, dg = torch.empty_like(x), torch.empty_like(x), torch.empty_like(gain)
    nscratch = W.rmsnorm_reverse_scratch(f32, m, n)
    # long rows: the shared-row softmax kernels with their slot-clearing kernel inside the graph
    lm, ln = 8, 50257
    logits = 3 * rnd(lm, ln)
    p, dp, dl = torch.empty_like(logits), rnd(lm, ln), torch.empty_like(logits)
    fs, rs = W.softmax_scratch(f32, lm, ln), W.softmax_reverse_scratch(f32, lm, ln)
    assert fs is not None and rs is not None
    # RMSNorm over the same long rows: the shared-row forward and the pipelined shared-row reverse
    lgain = 1 + 0.02 * rnd(ln)
    ly, ldx, ldg = torch.empty_like(logits), torch.empty_like(logits), torch.empty_like(lgain)
    lf, lr = W.rmsnorm_scratch(f32, lm, ln), W.rmsnorm_reverse_scratch(f32, lm, ln)
    assert lf is not None
    # column sums of a tall matrix through a workspace (partial rows, then the fixed-order finish)
    tall = rnd(3000, 512)
    sums = torch.empty(512, device="cuda", dtype=f32)
    kernels, _ = G.lib()
    cs = torch.empty(max(int(kernels.mpReduceScratchBytes(G.KEY[f32], 3000, 512)), 16), dtype=torch.uint8, device="cuda")
    a, b, c, d = (torch.rand(10007, generator=gen, device="cuda", dtype=f32) * 4 - 2 for _ in range(4))
    e = torch.empty_like(a)
    # an expression compiled at run time: its first (eager) call compiles and loads it, which a
    # capture could not do; after that a call is one kernel launch like any other
    chain = "relu(mul(sub(0,1),add(2,3)))"
    e2, up = torch.empty_like(a), rnd(10007)
    grads = [torch.empty_like(a) for _ in range(4)]
    for t in (x, gain, dy, y, dx, dg, logits, p, dp, dl, a, b, c, d, e, e2, up, *grads):
        assert t.dtype == f32

    # the entry point that brings its own workspace: its first (eager) call looks the built-in array up
    dx_na, dg_na = torch.empty_like(x), torch.empty_like(gain)

    def sequence():
        W.rmsnorm_forward(x, gain, y, 1e-6)
        W.rmsnorm_reverse(x, gain, dy, dx, dg, nscratch, 1e-6)
        assert kernels.mpRmsnormReverseR32NoAlloc(x.data_ptr(), gain.data_ptr(), dy.data_ptr(), dx_na.data_ptr(),
                                                  dg_na.data_ptr(), 1e-6, 0.0, m, n, W._ctx()) == 0
        W.softmax_forward(logits, p, fs)
        W.softmax_reverse(p, dp, dl, 0.0, rs)
        W.rmsnorm_forward(logits, lgain, ly, 1e-6, lf)
        W.rmsnorm_reverse(logits, lgain, dp, ldx, ldg, lr, 1e-6)
        W._launch("reduce_ij_j_scratch", f32, tall.data_ptr(), sums.data_ptr(), cs.data_ptr(), 0.0, 3000, 512)
        W.fused_forward(a, b, c, d, e)
        assert G.chain_forward(chain, [a, b, c, d], e2) == 0, G.chain_error()
        assert G.chain_reverse(chain, [a, b, c, d], up, grads, 0.0) == 0, G.chain_error()

    outputs = (y, dx, dg, dx_na, dg_na, p, dl, ly, ldx, ldg, sums, e, e2, *grads)
    G.say("eager sequence")
    sequence()
    torch.cuda.synchronize()
    eager = [t.clone() for t in outputs]
    graph = torch.cuda.CUDAGraph()
    G.say("capture")
    with torch.cuda.graph(graph):
        sequence()
    for replay in range(4):
        for t in outputs:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        G.say(f"replay {replay}")
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(outputs, eager):
            assert torch.equal(got, ref), f"replay {replay} differs from the eager result"
        assert torch.equal(dx_na, dx) and torch.equal(dg_na, dg), "the no-alloc entry point differs from the launcher"
        # eager work of the program between replays
        W.softmax_forward(logits, p, fs)
        torch.cuda.synchronize()
