"""The C++ host side (graph, op modules, deferred-elementwise fusion) on a GPU: runs
metaphor_amd/lib/host_check, which replays the reference's subgraphs example with its own
assertions and asserts one kernel per direction for the fused chain, then checks the tensors it
wrote against the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest
import torch

import gpu_lib as G
import oracle_lib as O
from metaphor_amd import ffi

pytestmark = pytest.mark.gpu


def _load(d, name, shape=None):
    a = np.fromfile(os.path.join(d, name + ".bin"), dtype=np.float32)
    return a.reshape(shape) if shape else a


def _cmp(got, ref, what, **kw):
    G.compare(torch.from_numpy(got), ref, torch.float32, what, **kw)


def test_host_library_end_to_end(tmp_path):
    exe = os.path.join(ffi.LIB_DIR, "host_check")
    assert os.path.exists(exe), "host_check is not built; run python -m metaphor_amd.kernelgen"
    G.say("host_check (C++ graph / ops / fusion)")
    res = subprocess.run([exe, str(tmp_path)], capture_output=True, text=True, timeout=120)
    print(res.stdout, res.stderr)
    assert res.returncode == 0, res.stderr
    assert "one kernel forward, one kernel reverse" in res.stdout
    d = str(tmp_path)

    a, b, c, dd = (_load(d, f"fused_{k}") for k in "abcd")
    ones = np.ones_like(a)
    _cmp(_load(d, "fused_e"), O.fused_selu_hadamard_add_add(a, b, c, dd), "host fused e", rowwise=False)
    _cmp(_load(d, "eval_e"), O.fused_selu_hadamard_add_add(a, b, c, dd), "host eval e", rowwise=False)
    refs = O.fused_selu_hadamard_add_add_reverse(a, b, c, dd, ones)
    for k, ref in zip("abcd", refs):
        _cmp(_load(d, f"fused_d{k}"), ref, f"host fused d{k}", rowwise=False)
    _cmp(_load(d, "fused_da2"), 2.0 * refs[0], "host fused da accumulated twice", rowwise=False)

    # the repeated-input expression runs per op: f = selu((a+a)*(c+d)); df/da = 2 * g * v
    u, v = O.addition(a, a), O.addition(c, dd)
    w = O.hadamard(u.astype(np.float32), v.astype(np.float32))
    _cmp(_load(d, "rep_f"), O.selu(w.astype(np.float32)), "host repeated-input f", rowwise=False, rtol=2e-5)
    g = O.selu_reverse(w, np.ones_like(w))
    _cmp(_load(d, "rep_da"), 2.0 * g * v, "host repeated-input da", rowwise=False, rtol=2e-5)
    _cmp(_load(d, "rep_dc"), g * u, "host repeated-input dc", rowwise=False, rtol=2e-5)

    # other generated chains (fp64 compositions of the pinned oracle pieces; upstream gradient = 1)
    a64, b64, c64, d64 = (z.astype(np.float64) for z in (a, b, c, dd))
    u, v = a64 + b64, c64 + d64
    _cmp(_load(d, "chain_mul_add_add"), u * v, "chain mul(add,add)", rowwise=False)
    _cmp(_load(d, "chain_mul_add_add_da"), v, "chain mul(add,add) da", rowwise=False)
    _cmp(_load(d, "chain_mul_add_add_dd"), u, "chain mul(add,add) dd", rowwise=False)
    w = (a64 - b64) * c64
    slope = O.selu_reverse(w, np.ones_like(w))
    _cmp(_load(d, "chain_selu_mul_sub"), O.selu(w), "chain selu(mul(sub,c))", rowwise=False)
    _cmp(_load(d, "chain_selu_mul_sub_da"), slope * c64, "chain selu(mul(sub,c)) da", rowwise=False)
    _cmp(_load(d, "chain_selu_mul_sub_db"), -slope * c64, "chain selu(mul(sub,c)) db", rowwise=False)
    _cmp(_load(d, "chain_selu_mul_sub_dc"), slope * (a64 - b64), "chain selu(mul(sub,c)) dc", rowwise=False,
         scale=np.abs(slope) * (np.abs(a64) + np.abs(b64)))
    sa = O.selu(a64 + b64)
    _cmp(_load(d, "chain_relu_selu_add"), O.relu(sa), "relu(selu(add))", rowwise=False)
    sa32 = _load(d, "chain_relu_selu_add")  # the eager relu saw the r32 selu output
    _cmp(_load(d, "chain_relu_selu_add_da"),
         O.selu_reverse(a64 + b64, np.ones_like(a64)) * (O.selu(a64 + b64) >= 0), "relu(selu(add)) da",
         rowwise=False)
    del sa32
    _cmp(_load(d, "plain_sub"), a64 - b64, "sub", rowwise=False)
    assert np.all(_load(d, "plain_sub_da") == 1.0) and np.all(_load(d, "plain_sub_db") == -1.0)

    m, n, eps = 37, 1000, 1e-6
    x, gain, dy = _load(d, "row_x", (m, n)), _load(d, "row_g"), _load(d, "row_dy", (m, n))
    _cmp(_load(d, "row_y", (m, n)), O.rmsnorm_ij_j(x, gain, eps), "host rmsnorm y")
    rdx, rdg = O.rmsnorm_ij_j_reverse(x, gain, dy, eps)
    sdx, sdg = G.rmsnorm_reverse_scales(x, gain, dy, eps)
    _cmp(_load(d, "row_dx", (m, n)), rdx, "host rmsnorm dx", scale=sdx)
    _cmp(_load(d, "row_dg"), rdg, "host rmsnorm dg", rowwise=False, scale=sdg)

    s, dp = _load(d, "row_s", (m, n)), _load(d, "row_dp", (m, n))
    p = _load(d, "row_p", (m, n))
    s2 = O.addition(s, s).astype(np.float32)
    _cmp(p, O.softmax_ij_j(s2), "host softmax(s+s)", atol=1e-6)
    dz = O.softmax_ij_j_reverse(p, dp)
    _cmp(_load(d, "row_ds", (m, n)), 2.0 * dz, "host d softmax(s+s) / ds",
         scale=2.0 * G.softmax_reverse_scale(p, dp))
