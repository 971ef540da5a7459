"""The entry point that allocates nothing: mpRmsnormReverseR32NoAlloc against
launch_rmsnorm_ij_j_reverse_r32 (the entry point it is a variant of), through the C ABI.

Both run the same kernels, the first on the library's built-in device array and the second on a
caller-owned workspace, so the results must agree bit for bit (tighter than the r32 bar of 1e-5
relative that the launcher itself is held to against the oracle). Two calls in a row, the second
on a smaller input: the array keeps the first call's contents and nothing may leak from them.
"""
import contextlib
import io
import os

import numpy as np
import pytest
import torch

import gpu_lib as G
import oracle_lib as O
from metaphor_amd import ffi

pytestmark = pytest.mark.gpu
F32 = torch.float32


def _inputs(m, n, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, n)).astype(np.float32)
    g = (1.0 + 0.02 * rng.standard_normal(n)).astype(np.float32)
    dy = rng.standard_normal((m, n)).astype(np.float32)
    return x, g, dy


def _run_both(m, n, seed, alpha=0.0):
    kernels, _ = G.lib()
    x, g, dy = _inputs(m, n, seed)
    eps = 1e-6
    dx0 = np.random.default_rng(seed + 1).standard_normal((m, n)).astype(np.float32)
    dg0 = np.random.default_rng(seed + 2).standard_normal(n).astype(np.float32)
    xd, gd, dyd = G.dev(x, F32), G.dev(g, F32), G.dev(dy, F32)
    # existing entry point, caller-owned workspace
    dx_a, dg_a = G.dev(dx0, F32), G.dev(dg0, F32)
    scratch, _ = G.rmsnorm_scratch(F32, m, n)
    G.say(f"rmsnorm reverse with caller scratch r32 [{m},{n}] alpha {alpha}")
    G.rmsnorm_reverse(xd.t, gd.t, dyd.t, dx_a.t, dg_a.t, scratch.t, eps, alpha)
    # the variant without the scratch argument
    dx_b, dg_b = G.dev(dx0, F32), G.dev(dg0, F32)
    G.say(f"mpRmsnormReverseR32NoAlloc [{m},{n}] alpha {alpha}")
    rc = kernels.mpRmsnormReverseR32NoAlloc(xd.t.data_ptr(), gd.t.data_ptr(), dyd.t.data_ptr(), dx_b.t.data_ptr(),
                                            dg_b.t.data_ptr(), eps, float(alpha), m, n, G.ctx())
    assert rc == 0
    torch.cuda.synchronize()
    for t, what in ((dx_a, "dx (scratch)"), (dg_a, "dg (scratch)"), (dx_b, "dx (no alloc)"), (dg_b, "dg (no alloc)"),
                    (scratch, "scratch")):
        t.check(what)
    assert torch.equal(dx_a.t, dx_b.t), "dx differs between the two entry points"
    assert torch.equal(dg_a.t, dg_b.t), "dgain differs between the two entry points"
    # and both against the oracle, at the launcher's own bar
    dx_ref, dg_ref = O.rmsnorm_ij_j_reverse(x, g, dy, eps, dx_in=dx0, dg_in=dg0, alpha=alpha) if alpha else \
        O.rmsnorm_ij_j_reverse(x, g, dy, eps)
    sdx, sdg = G.rmsnorm_reverse_scales(x, g, dy, eps, dx0 if alpha else None, dg0 if alpha else None, alpha)
    G.compare(dx_b.t, dx_ref, F32, f"no-alloc dx [{m},{n}]", scale=sdx)
    G.compare(dg_b.t, dg_ref, F32, f"no-alloc dgain [{m},{n}]", rowwise=False, scale=sdg)


def test_two_calls_in_a_row_second_smaller():
    _run_both(1024, 4096, seed=11)   # one partial row per workgroup, 512 workgroups' worth of rows
    _run_both(96, 1000, seed=12)     # fewer and shorter partial rows: the array still holds the first call's


def test_accumulating_call_and_shared_long_rows():
    _run_both(64, 4096, seed=13, alpha=1.0)
    _run_both(40, 40000, seed=14)    # rows shared by several workgroups: their exchange words live in the array too


def test_rejects_what_the_array_cannot_hold():
    kernels, _ = G.lib()
    m, n = 4096, 16384                # 512 partial rows of 64 KiB: 32 MiB
    need = int(kernels.mpRmsnormReverseScratchBytes(ffi.R32, m, n))
    assert need > 16 << 20
    dx = G.Guarded((8,), F32)
    G.say("mpRmsnormReverseR32NoAlloc beyond the array: must refuse and enqueue nothing")
    rc = kernels.mpRmsnormReverseR32NoAlloc(None, None, None, dx.t.data_ptr(), None, 1e-6, 0.0, m, n, G.ctx())
    assert rc == 1
    torch.cuda.synchronize()
    dx.check("refused call")
