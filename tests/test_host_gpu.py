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

    # the same repeated-input shape on a graph that fuses at run time: f = selu((a+a)*(c-d)), one kernel
    # per direction (host_check asserts the launch counts); da = 2*g*v, dc = g*u, dd = -g*u
    ua, va = 2.0 * a.astype(np.float64), c.astype(np.float64) - dd.astype(np.float64)
    wa = ua * va
    ga_ = O.selu_reverse(wa, np.ones_like(wa))
    _cmp(_load(d, "any_f"), O.selu(wa), "run-time chain f", rowwise=False, scale=np.abs(wa))
    _cmp(_load(d, "any_da"), 2.0 * ga_ * va, "run-time chain da", rowwise=False)
    _cmp(_load(d, "any_dc"), ga_ * ua, "run-time chain dc", rowwise=False)
    _cmp(_load(d, "any_dd"), -ga_ * ua, "run-time chain dd", rowwise=False)
    _cmp(_load(d, "any_da2"), 4.0 * ga_ * va, "run-time chain da accumulated twice", rowwise=False)
    _cmp(_load(d, "any_sub"), va, "single op on a fusing graph", rowwise=False)
    # relu(0.125 * (a * c) + 0.5) with its constants inside the kernel; upstream gradient = 1
    a64_, c64_ = a.astype(np.float64), c.astype(np.float64)
    pre = 0.125 * (a64_ * c64_) + 0.5
    on = (pre >= 0).astype(np.float64)
    _cmp(_load(d, "any_affine"), np.where(pre >= 0, pre, 0.0), "run-time chain with constants", rowwise=False)
    _cmp(_load(d, "any_affine_da"), on * 0.125 * c64_, "run-time chain with constants da", rowwise=False)
    _cmp(_load(d, "any_affine_dc"), on * 0.125 * a64_, "run-time chain with constants dc", rowwise=False)
    # the same kernel with other constants (host_check asserts that nothing was compiled for it)
    pre2 = -0.75 * (a64_ * c64_) + 0.25
    on2 = (pre2 >= 0).astype(np.float64)
    _cmp(_load(d, "any_affine2"), np.where(pre2 >= 0, pre2, 0.0), "run-time chain, other constants", rowwise=False)
    _cmp(_load(d, "any_affine2_da"), on2 * -0.75 * c64_, "run-time chain, other constants da", rowwise=False)
    _cmp(_load(d, "any_affine2_dc"), on2 * -0.75 * a64_, "run-time chain, other constants dc", rowwise=False)

    # two results out of one forward kernel: u = a + b; e1 = selu(u * c); e2 = relu(u - d); each reversed
    # with an upstream gradient of 1, the leaf gradients accumulate over the two reverses
    b64_, d64_ = b.astype(np.float64), dd.astype(np.float64)
    u_ = a64_ + b64_
    w1, w2 = u_ * c64_, u_ - d64_
    g1 = O.selu_reverse(w1, np.ones_like(w1))
    g2 = (w2 >= 0).astype(np.float64)
    _cmp(_load(d, "two_e1"), O.selu(w1), "two results e1", rowwise=False, scale=np.abs(w1))
    _cmp(_load(d, "two_e2"), np.where(w2 >= 0, w2, 0.0), "two results e2", rowwise=False)
    _cmp(_load(d, "two_da"), g1 * c64_ + g2, "two results da", rowwise=False)
    _cmp(_load(d, "two_db"), g1 * c64_ + g2, "two results db", rowwise=False)
    _cmp(_load(d, "two_dc"), g1 * u_, "two results dc", rowwise=False)
    _cmp(_load(d, "two_dd"), -g2, "two results dd", rowwise=False)

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
    w4 = (a64 + b64) * (c64 + dd.astype(np.float64))
    _cmp(_load(d, "chain_relu_mul_add_add"), np.maximum(w4, 0.0), "relu(mul(add,add))", rowwise=False)
    live = (_load(d, "chain_relu_mul_add_add") > 0).astype(np.float64)  # the slope the r32 kernel saw
    _cmp(_load(d, "chain_relu_mul_add_add_da"), live * (c64 + dd.astype(np.float64)), "relu(mul(add,add)) da",
         rowwise=False, rtol=2e-5)
    _cmp(_load(d, "chain_relu_mul_add_add_dc"), live * (a64 + b64), "relu(mul(add,add)) dc", rowwise=False, rtol=2e-5)
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

    # ---- matrix side: every inner-product expression with its two gradients
    assert "inner products, permutate, reduce / broadcast, checkpoint files ok" in res.stdout
    m, n, k = 37, 53, 29
    a, b, bt, at = _load(d, "mx_a", (m, n)), _load(d, "mx_b", (n, k)), _load(d, "mx_bt", (k, n)), _load(d, "mx_at", (n, m))
    v, u = _load(d, "mx_v"), _load(d, "mx_u")
    g, gi, gn = _load(d, "mx_g", (m, k)), _load(d, "mx_gi", (m, 1)), _load(d, "mx_gn", (1, n))

    def prod(x, y, alpha, ta=False, tb=False):
        return O.inner_product(x, y, alpha, ta=ta, tb=tb, with_scale=True)

    def check(name, z, dx, dy):
        for suffix, (ref, scale) in (("z", z), ("dx", dx), ("dy", dy)):
            got = _load(d, f"mx_{name}_{suffix}")
            _cmp(got.reshape(ref.shape), ref, f"host inner product {name} {suffix}", rowwise=False, scale=scale)

    check("nn", prod(a, b, 1.0), prod(g, b, 1.0, tb=True), prod(a, g, 1.0, ta=True))
    check("nt", prod(a, bt, 0.5, tb=True), prod(g, bt, 0.5), prod(g, a, 0.5, ta=True))
    check("tn", prod(at, b, -2.0, ta=True), prod(b, g, -2.0, tb=True), prod(at, g, -2.0))
    vcol, urow = v.reshape(n, 1), u.reshape(1, m)
    check("mv", prod(a, vcol, 1.0), prod(gi, vcol, 1.0, tb=True), prod(a, gi, 1.0, ta=True))
    check("vm", prod(urow, a, 1.5), prod(gn, a, 1.5, tb=True), prod(urow, gn, 1.5, ta=True))
    ref, scale = prod(g, b, 1.0, tb=True)
    _cmp(_load(d, "mx_nn_dx2", (m, n)), 2.0 * ref, "host inner product gradient accumulated twice", rowwise=False,
         scale=2.0 * scale)
    # the saved checkpoint files are the raw bytes of the weights, in creation order after the example's two
    assert np.array_equal(np.fromfile(os.path.join(d, "single_a"), dtype=np.float32), a.ravel())
    assert np.array_equal(np.fromfile(os.path.join(d, "ckpt_0"), dtype=np.float32), [1, 2, 3, 4, 5, 6])
    assert np.array_equal(np.fromfile(os.path.join(d, "ckpt_2"), dtype=np.float32), a.ravel())
    assert np.array_equal(np.fromfile(os.path.join(d, "ckpt_7"), dtype=np.float32), u)
    # permutate(dilate(translate(a, 0.25), 3)) and its gradient
    t = O.dilate(O.translate(a, 0.25).astype(np.float32), 3.0)
    _cmp(_load(d, "mx_perm", (n, m)), O.permutate_ij_ji(t.astype(np.float32)), "host permutate chain", rowwise=False)
    _cmp(_load(d, "mx_perm_da", (m, n)), 3.0 * O.permutate_ij_ji(at), "host permutate chain da", rowwise=False)
    # reduce / broadcast and their reverses
    _cmp(_load(d, "mx_reduce_i"), O.reduce_ij_i(a), "host reduce ij->i", rowwise=False,
         scale=np.abs(a.astype(np.float64)).sum(1))
    _cmp(_load(d, "mx_reduce_i_da", (m, n)), O.broadcast_i_ij(gi.ravel(), m, n), "host reduce reverse", rowwise=False)
    gmn = _load(d, "mx_gmn", (m, n))
    _cmp(_load(d, "mx_bcast_j", (m, n)), O.broadcast_j_ij(v, m, n), "host broadcast j->ij", rowwise=False)
    _cmp(_load(d, "mx_bcast_j_dv"), O.reduce_ij_j(gmn), "host broadcast reverse", rowwise=False,
         scale=np.abs(gmn.astype(np.float64)).sum(0))
