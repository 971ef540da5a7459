"""Two streams of the library at once: launchers keep no state that streams share (each stream
context owns its workspace, every other scratch buffer belongs to the caller), so two sequences
enqueued side by side, with nothing but their own stream order, give the oracle's results."""
import numpy as np
import pytest
import torch

import gpu_lib as G
import oracle_lib as O

pytestmark = pytest.mark.gpu

F32 = torch.float32


def _bytes(n):
    return torch.empty(max(int(n), 16), dtype=torch.uint8, device="cuda")


def test_two_streams_run_side_by_side():
    kernels, _ = G.lib()
    r = np.random.default_rng(71)
    eps = 1e-6
    jobs = []
    # per stream: its own shapes, operands and caller-owned scratch (long rows take the shared-row kernels)
    for (m, n, tall) in ((48, 70000, (30000, 96)), (40, 66000, (26000, 128))):
        x = G.dev(r.normal(0, 1, (m, n)), F32)
        g = G.dev(r.normal(1, 0.02, n), F32)
        dy = G.dev(r.normal(0, 1, (m, n)), F32)
        t = G.dev(r.normal(0, 1, tall), F32)
        jobs.append(dict(
            m=m, n=n, x=x, g=g, dy=dy, t=t,
            y=G.Guarded((m, n), F32), p=G.Guarded((m, n), F32), dx=G.Guarded((m, n), F32), dg=G.Guarded((n,), F32),
            sums=G.Guarded((tall[1],), F32),
            s_norm=_bytes(kernels.mpRmsnormScratchBytes(G.KEY[F32], m, n)),
            s_rev=_bytes(kernels.mpRmsnormReverseScratchBytes(G.KEY[F32], m, n)),
            s_soft=_bytes(kernels.mpSoftmaxScratchBytes(G.KEY[F32], m, n))))
    with G.BlasStream() as s0, G.BlasStream() as s1:
        torch.cuda.synchronize()
        G.say("rmsnorm forward + reverse, softmax and column sums on two streams at once")
        for _ in range(3):  # the same work three times over: later launches reuse the scratch of earlier ones
            for stream, j in ((s0, jobs[0]), (s1, jobs[1])):
                m, n = j["m"], j["n"]
                stream.enqueue("rmsnorm_ij_j", F32, j["x"].t.data_ptr(), j["g"].t.data_ptr(), j["y"].t.data_ptr(),
                               j["s_norm"].data_ptr(), eps, m, n)
                stream.enqueue("softmax_ij_j", F32, j["x"].t.data_ptr(), j["p"].t.data_ptr(), j["s_soft"].data_ptr(), m, n)
                stream.enqueue("rmsnorm_ij_j_reverse", F32, j["x"].t.data_ptr(), j["g"].t.data_ptr(), j["dy"].t.data_ptr(),
                               j["dx"].t.data_ptr(), j["dg"].t.data_ptr(), j["s_rev"].data_ptr(), eps, 0.0, m, n)
                stream.enqueue("reduce_ij_j", F32, j["t"].t.data_ptr(), j["sums"].t.data_ptr(), 0.0, *j["t"].t.shape)
        s0.sync()
        s1.sync()
    for k, j in enumerate(jobs):
        xh, gh, dyh = G.host(j["x"].t), G.host(j["g"].t), G.host(j["dy"].t)
        G.compare(j["y"].t, O.rmsnorm_ij_j(xh, gh, eps), F32, f"stream {k} rmsnorm")
        G.compare(j["p"].t, O.softmax_ij_j(xh), F32, f"stream {k} softmax", **G.softmax_tol(F32))
        rdx, rdg = O.rmsnorm_ij_j_reverse(xh, gh, dyh, eps)
        sdx, sdg = G.rmsnorm_reverse_scales(xh, gh, dyh, eps)
        G.compare(j["dx"].t, rdx, F32, f"stream {k} rmsnorm reverse dx", scale=sdx)
        G.compare(j["dg"].t, rdg, F32, f"stream {k} rmsnorm reverse dg", rowwise=False, scale=sdg)
        th = G.host(j["t"].t)
        G.compare(j["sums"].t, O.reduce_ij_j(th), F32, f"stream {k} column sums", rowwise=False,
                  scale=np.abs(th.astype(np.float64)).sum(axis=0))
        for name in ("x", "g", "dy", "t", "y", "p", "dx", "dg", "sums"):
            j[name].check(f"stream {k} {name}")
