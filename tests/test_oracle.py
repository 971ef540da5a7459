"""Pins the CPU oracle without the reference (which has no tests, no golden vectors and
cannot be built here): hand-computable answers from the reference's examples, fp64 library
routines (torch softmax / selu / rms_norm, torch autograd for every reverse), central finite
differences, and algebraic invariants. Each check is chosen so that a dropped term, a wrong
sign, a transposed operand or a mean-vs-sum slip fails it."""
import numpy as np
import pytest
import torch

import oracle_lib as O

torch.set_default_dtype(torch.float64)
RNG = np.random.default_rng(1234)


def t64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64).copy())


# ---------------------------------------------------------------- storage types

def test_half_conversion_exhaustive_roundtrip():
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float64)
    for b, v in zip(bits[::7], vals[::7]):
        got = O.half_bits_to_double(int(b))
        if np.isnan(v):
            assert np.isnan(got)
            continue
        assert got == v
        assert O.double_to_half_bits(v) == int(b)


def test_double_to_half_rounds_to_nearest_even_like_numpy():
    xs = np.concatenate([
        RNG.normal(0, 1, 2000), RNG.normal(0, 1e-5, 2000), RNG.normal(0, 3e4, 2000),
        np.array([65519.99, 65520.0, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -24 * 1.5,
                  2.0 ** -24 * 2.5, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, -0.0, 0.0]),
    ])
    want = xs.astype(np.float16).view(np.uint16)
    got = np.array([O.double_to_half_bits(x) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dt", [np.float16, np.float32, np.float64])
def test_inputs_are_read_in_their_storage_type(dt):
    a = RNG.normal(0, 1, 257).astype(dt)
    b = RNG.normal(0, 1, 257).astype(dt)
    assert np.array_equal(O.addition(a, b), a.astype(np.float64) + b.astype(np.float64))


# ---------------------------------------------------------------- elementwise

def test_known_answers_from_reference_examples():
    # src/examples/subgraphs.zig:34-45 — ones through add twice: 2 then 3.
    one = np.ones(32, dtype=np.float32)
    z1 = O.addition(one, one)
    assert np.all(z1 == 2.0)
    assert np.all(O.addition(z1.astype(np.float32), one) == 3.0)
    # src/examples/experimental.zig:19-34 — x=[[1,2],[3,4],[5,6]], y=[[1,2],[3,4]].
    x = np.array([[1, 2], [3, 4], [5, 6]], dtype=np.float32)
    y = np.array([[1, 2], [3, 4]], dtype=np.float32)
    assert np.array_equal(O.reduce_ij_i(y), [3.0, 7.0])
    assert np.array_equal(O.reduce_ij_j(x), [9.0, 12.0])


def test_add_hadamard_and_accumulating_reverse():
    a = RNG.normal(0, 1, 1001).astype(np.float32)
    b = RNG.normal(0, 1, 1001).astype(np.float32)
    c0 = RNG.normal(0, 1, 1001).astype(np.float32)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    assert np.array_equal(O.addition(a, b), a64 + b64)
    assert np.array_equal(O.hadamard(a, b), a64 * b64)
    assert np.array_equal(O.hadamard_reverse(a, b), a64 * b64)
    assert np.array_equal(O.hadamard_reverse(a, b, c0), c0.astype(np.float64) + a64 * b64)


def test_remaining_elementwise_launchers_closed_forms():
    a = np.concatenate([RNG.normal(0, 1, 500), [0.0, -0.0]]).astype(np.float32)
    b = RNG.normal(0, 1, a.size).astype(np.float32)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    assert np.array_equal(O.subtraction(a, b), a64 - b64)
    assert np.array_equal(O.negate(a), -a64)
    assert np.array_equal(O.copy(a), a64)
    assert np.array_equal(O.relu(a), torch.relu(t64(a)).numpy())
    assert np.array_equal(O.stepwise(a), (a64 >= 0).astype(np.float64))
    assert O.stepwise(np.array([-0.0]))[0] == 1.0  # -0.0 >= 0, as in relu.cu:12
    # relu reverse: subgraphs.zig:34-45 — all-ones through relu(add) gives gradients of 1
    one = np.ones(8, dtype=np.float32)
    assert np.all(O.relu_reverse(O.addition(one, one).astype(np.float32), one) == 1.0)
    at = t64(a).requires_grad_(True)
    torch.relu(at).backward(t64(b))
    nz = a64 != 0  # torch takes 0 as the slope at exactly 0; the reference takes 1
    assert np.array_equal(O.relu_reverse(a, b)[nz], at.grad.numpy()[nz])
    assert np.array_equal(O.relu_reverse(a, b)[~nz], b64[~nz])
    assert np.array_equal(O.relu_reverse(a, b, b), b64 + O.relu_reverse(a, b))
    v = 0.1  # not representable: narrowed to the storage type before use
    assert np.array_equal(O.dilate(a, v), a64 * float(np.float32(v)))
    assert np.array_equal(O.translate(a, v), a64 + float(np.float32(v)))
    assert np.array_equal(O.dilate_reverse(a, v, b), b64 + a64 * float(np.float32(v)))
    h = a.astype(np.float16)
    assert np.array_equal(O.dilate(h, v), h.astype(np.float64) * float(np.float16(v)))
    assert np.array_equal(O.fill(np.float32, v, 5), np.full(5, float(np.float32(v))))
    assert np.array_equal(O.sequence(np.float64, 1.5, 0.25, 6), 1.5 + 0.25 * np.arange(6))


def test_reduce_blend_and_orientation():
    src = RNG.normal(0, 1, (5, 9))
    d_i, d_j = RNG.normal(0, 1, 5), RNG.normal(0, 1, 9)
    np.testing.assert_allclose(O.reduce_ij_i(src, d_i, 0.5), src.sum(1) + 0.5 * d_i, rtol=1e-14)
    np.testing.assert_allclose(O.reduce_ij_j(src, d_j, -2.0), src.sum(0) - 2.0 * d_j, rtol=1e-14)


def test_permutate_is_numpy_transpose_with_blend():
    src = RNG.normal(0, 1, (7, 13)).astype(np.float32)
    old = RNG.normal(0, 1, (13, 7)).astype(np.float32)
    assert np.array_equal(O.permutate_ij_ji(src), src.T.astype(np.float64))
    assert np.array_equal(O.permutate_ij_ji(O.permutate_ij_ji(src).astype(np.float32)), src.astype(np.float64))
    np.testing.assert_allclose(O.permutate_ij_ji(src, old, 1.0), src.T.astype(np.float64) + old, rtol=1e-15)
    np.testing.assert_allclose(O.permutate_ij_ji(src, old, -0.5), src.T.astype(np.float64) - 0.5 * old, rtol=1e-15)
    # a non-square index slip (cols used as the output stride) would move this single entry
    e = np.zeros((3, 5), dtype=np.float64)
    e[2, 1] = 1.0
    out = O.permutate_ij_ji(e)
    assert out.shape == (5, 3) and out[1, 2] == 1.0 and out.sum() == 1.0


def test_inner_product_known_answers_and_operand_forms():
    # src/examples/experimental.zig:19-34,51-62 — x = [[1,2],[3,4],[5,6]], y = [[1,2],[3,4]]:
    # z = x.y by hand; with a seed of ones the reverse gives dx = ones.T(y) (rows [3,7]) and
    # dy = T(x).ones (rows [9,9],[12,12]), the values the example prints as bn and dn.
    x = np.array([[1, 2], [3, 4], [5, 6]], dtype=np.float32)
    y = np.array([[1, 2], [3, 4]], dtype=np.float32)
    assert np.array_equal(O.inner_product(x, y), [[7, 10], [15, 22], [23, 34]])
    ones = np.ones((3, 2), dtype=np.float32)
    assert np.array_equal(O.inner_product(ones, y, tb=True), [[3, 7]] * 3)       # ij,kj->ik
    assert np.array_equal(O.inner_product(x, ones, ta=True), [[9, 9], [12, 12]])  # ji,jk->ik
    # library routine in fp64, every operand form, non-square everywhere
    m, n, k = 5, 7, 3
    a, b = RNG.normal(0, 1, (m, n)), RNG.normal(0, 1, (n, k))
    c0 = RNG.normal(0, 1, (m, k))
    ref = a @ b
    np.testing.assert_allclose(O.inner_product(a, b), ref, rtol=1e-13, atol=1e-14)
    np.testing.assert_allclose(O.inner_product(a, np.ascontiguousarray(b.T), tb=True), ref, rtol=1e-13, atol=1e-14)
    np.testing.assert_allclose(O.inner_product(np.ascontiguousarray(a.T), b, ta=True), ref, rtol=1e-13, atol=1e-14)
    np.testing.assert_allclose(O.inner_product(a, b, 0.5, c0, -2.0), 0.5 * ref - 2.0 * c0, rtol=1e-13, atol=1e-14)
    # identity and (A.B)^T = B^T.A^T
    np.testing.assert_allclose(O.inner_product(a, np.eye(n)), a, rtol=0)
    np.testing.assert_allclose(O.inner_product(np.ascontiguousarray(b.T), np.ascontiguousarray(a.T)), ref.T, rtol=1e-13, atol=1e-14)
    # the scale output is the same product over absolute values
    _, scale = O.inner_product(a, b, 0.5, c0, -2.0, with_scale=True)
    np.testing.assert_allclose(scale, 0.5 * (np.abs(a) @ np.abs(b)) + 2.0 * np.abs(c0), rtol=1e-13)
    # autograd of z = scale * x.y gives the reverse operand forms used by src/ops/inner_product.zig:305-326
    at, bt = t64(a).requires_grad_(True), t64(b).requires_grad_(True)
    gz = RNG.normal(0, 1, (m, k))
    (1.5 * at @ bt).backward(t64(gz))
    np.testing.assert_allclose(O.inner_product(gz, b, 1.5, tb=True), at.grad.numpy(), rtol=1e-13, atol=1e-14)
    np.testing.assert_allclose(O.inner_product(a, gz, 1.5, ta=True), bt.grad.numpy(), rtol=1e-13, atol=1e-14)
    # half inputs are read exactly
    ah, bh = a.astype(np.float16), b.astype(np.float16)
    np.testing.assert_allclose(O.inner_product(ah, bh), ah.astype(np.float64) @ bh.astype(np.float64), rtol=1e-13, atol=1e-14)


def test_broadcasts_are_the_reverses_of_the_reductions():
    m, n = 5, 9
    src_i, src_j = RNG.normal(0, 1, m), RNG.normal(0, 1, n)
    old = RNG.normal(0, 1, (m, n))
    np.testing.assert_allclose(O.broadcast_i_ij(src_i, m, n), np.repeat(src_i[:, None], n, 1), rtol=0)
    np.testing.assert_allclose(O.broadcast_j_ij(src_j, m, n), np.repeat(src_j[None, :], m, 0), rtol=0)
    np.testing.assert_allclose(O.broadcast_i_ij(src_i, m, n, old, 1.0), src_i[:, None] + old, rtol=1e-15)
    np.testing.assert_allclose(O.broadcast_j_ij(src_j, m, n, old, 0.5), src_j[None, :] + 0.5 * old, rtol=1e-15)
    # autograd: d(sum_j x_ij)/dx = broadcast of the upstream gradient over j
    xt = t64(old).requires_grad_(True)
    xt.sum(dim=1).backward(t64(src_i))
    np.testing.assert_allclose(O.broadcast_i_ij(src_i, m, n), xt.grad.numpy(), rtol=0)
    xt = t64(old).requires_grad_(True)
    xt.sum(dim=0).backward(t64(src_j))
    np.testing.assert_allclose(O.broadcast_j_ij(src_j, m, n), xt.grad.numpy(), rtol=0)


def test_selu_closed_form_and_library():
    x = np.concatenate([RNG.uniform(-20, 20, 4000), [0.0, -0.0, 1e-12, -1e-12, -745.0, 700.0]])
    got = O.selu(x)
    want = torch.nn.functional.selu(t64(x)).numpy()
    # the library uses the full-precision constants; this workload truncates them to 8 digits
    np.testing.assert_allclose(got, want, rtol=4e-8, atol=0)
    lam, alp = 1.0507010, 1.6732632
    assert O.selu(np.array([0.0]))[0] == 0.0
    assert O.selu(np.array([3.0]))[0] == lam * 3.0
    np.testing.assert_allclose(O.selu(np.array([-800.0]))[0], -lam * alp, rtol=1e-15)
    # expm1 (not exp-1): relative accuracy survives near 0-
    np.testing.assert_allclose(O.selu(np.array([-1e-10]))[0], lam * alp * -1e-10, rtol=1e-9)


def test_selu_reverse_vs_autograd_and_accumulation():
    x = np.concatenate([RNG.uniform(-6, 6, 2000), [0.0]])
    gy = RNG.normal(0, 1, x.size)
    g0 = RNG.normal(0, 1, x.size)
    xt = t64(x).requires_grad_(True)
    torch.nn.functional.selu(xt).backward(t64(gy))
    np.testing.assert_allclose(O.selu_reverse(x, gy), xt.grad.numpy(), rtol=6e-8, atol=0)
    np.testing.assert_allclose(O.selu_reverse(x, gy, g0), g0 + O.selu_reverse(x, gy), rtol=1e-15)
    # at exactly 0 the expm1 branch is taken: derivative scale*alpha
    assert O.selu_reverse(np.array([0.0]), np.array([1.0]))[0] == 1.0507010 * 1.6732632


def test_fused_chain_equals_composition_and_autograd():
    n = 3001
    a, b, c, d = (RNG.uniform(-2, 2, n).astype(np.float32) for _ in range(4))
    de = RNG.normal(0, 1, n).astype(np.float32)
    e = O.fused_selu_hadamard_add_add(a, b, c, d)
    u, v = O.addition(a, b), O.addition(c, d)
    assert np.array_equal(e, O.selu(O.hadamard(u, v)))
    ts = [t64(z).requires_grad_(True) for z in (a, b, c, d)]
    out = torch.nn.functional.selu((ts[0] + ts[1]) * (ts[2] + ts[3]))
    np.testing.assert_allclose(e, out.detach().numpy(), rtol=4e-8)
    out.backward(t64(de))
    da, db, dc, dd = O.fused_selu_hadamard_add_add_reverse(a, b, c, d, de)
    for got, t in zip((da, db, dc, dd), ts):
        np.testing.assert_allclose(got, t.grad.numpy(), rtol=6e-8, atol=1e-300)
    assert np.array_equal(da, db) and np.array_equal(dc, dd)
    # blend: out = val + alpha*in
    gin = tuple(RNG.normal(0, 1, n).astype(np.float32) for _ in range(4))
    outs = O.fused_selu_hadamard_add_add_reverse(a, b, c, d, de, gin, alpha=1.0)
    for o, base, g in zip(outs, (da, db, dc, dd), gin):
        np.testing.assert_allclose(o, base + g.astype(np.float64), rtol=1e-15)


def test_fused_reverse_central_difference():
    a, b, c, d = (RNG.uniform(-2, 2, 64) for _ in range(4))
    de = np.ones(64)
    da, _, dc, _ = O.fused_selu_hadamard_add_add_reverse(a, b, c, d, de)
    h = 1e-6
    fd_a = (O.fused_selu_hadamard_add_add(a + h, b, c, d) - O.fused_selu_hadamard_add_add(a - h, b, c, d)) / (2 * h)
    fd_c = (O.fused_selu_hadamard_add_add(a, b, c + h, d) - O.fused_selu_hadamard_add_add(a, b, c - h, d)) / (2 * h)
    w = (a + b) * (c + d)
    ok = np.abs(w) > 1e-4  # away from the kink of selu' at 0
    np.testing.assert_allclose(da[ok], fd_a[ok], rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(dc[ok], fd_c[ok], rtol=1e-6, atol=1e-8)


# ---------------------------------------------------------------- softmax

def _causal(x):
    x = x.copy()
    r, c = np.indices(x.shape)
    x[c > r] = -np.inf
    return x


def test_softmax_vs_library_and_invariants():
    x = 4.0 * RNG.normal(0, 1, (37, 1000))
    y = O.softmax_ij_j(x)
    np.testing.assert_allclose(y, torch.softmax(t64(x), dim=-1).numpy(), rtol=1e-13, atol=1e-300)
    np.testing.assert_allclose(y.sum(1), 1.0, rtol=1e-13)
    shift = RNG.normal(0, 10, (37, 1))
    np.testing.assert_allclose(O.softmax_ij_j(x + shift), y, rtol=1e-11)
    # orientation: rows, not columns
    assert abs(y.sum(0)[0] - 1.0) > 1e-3
    # brute force on a tiny row
    r = np.array([[1.0, 2.0, 3.0]])
    e = np.exp(r - 3.0)
    np.testing.assert_allclose(O.softmax_ij_j(r), e / e.sum(), rtol=1e-15)


def test_softmax_masked_rows_and_degenerate_lengths():
    x = _causal(RNG.normal(0, 2, (16, 16)))
    y = O.softmax_ij_j(x)
    assert np.all(y[np.isinf(x)] == 0.0)
    assert y[0, 0] == 1.0  # single finite entry
    np.testing.assert_allclose(y.sum(1), 1.0, rtol=1e-14)
    np.testing.assert_allclose(y, torch.softmax(t64(x), dim=-1).numpy(), rtol=1e-13)
    assert np.all(O.softmax_ij_j(RNG.normal(0, 1, (5, 1))) == 1.0)
    x16 = _causal(RNG.normal(0, 2, (8, 8))).astype(np.float16)
    np.testing.assert_allclose(O.softmax_ij_j(x16), torch.softmax(t64(x16), dim=-1).numpy(), rtol=1e-13)
    # large spread never overflows
    big = np.array([[1000.0, -1000.0, 999.0]])
    assert np.isfinite(O.softmax_ij_j(big)).all()


def test_softmax_reverse_vs_autograd_and_invariants():
    x = _causal(RNG.normal(0, 2, (24, 24)))
    dy = RNG.normal(0, 1, x.shape)
    xt = t64(x).requires_grad_(True)
    yt = torch.softmax(xt, dim=-1)
    yt.backward(t64(dy))
    y = yt.detach().numpy()
    dx = O.softmax_ij_j_reverse(y, dy)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-12, atol=1e-16)
    np.testing.assert_allclose(dx.sum(1), 0.0, atol=1e-14)
    assert np.all(dx[y == 0.0] == 0.0)
    dx0 = RNG.normal(0, 1, x.shape)
    np.testing.assert_allclose(O.softmax_ij_j_reverse(y, dy, dx0, 1.0), dx + dx0, rtol=1e-14, atol=1e-16)
    np.testing.assert_allclose(O.softmax_ij_j_reverse(y, dy, dx0, 0.25), dx + 0.25 * dx0, rtol=1e-14, atol=1e-16)


def test_softmax_reverse_jacobian_by_finite_differences():
    x = RNG.normal(0, 1, (1, 6))
    y = O.softmax_ij_j(x)
    h = 1e-6
    J = np.zeros((6, 6))
    for k in range(6):
        xp, xm = x.copy(), x.copy()
        xp[0, k] += h
        xm[0, k] -= h
        J[:, k] = (O.softmax_ij_j(xp) - O.softmax_ij_j(xm))[0] / (2 * h)
    for k in range(6):
        dy = np.zeros((1, 6))
        dy[0, k] = 1.0
        # dx = J^T dy
        np.testing.assert_allclose(O.softmax_ij_j_reverse(y, dy)[0], J[k, :], rtol=1e-6, atol=1e-9)


# ---------------------------------------------------------------- RMSNorm

def test_rmsnorm_vs_library_and_invariants():
    m, n, eps = 19, 515, 1e-6
    x = RNG.normal(0, 1, (m, n))
    g = RNG.normal(1, 0.02, n)
    y = O.rmsnorm_ij_j(x, g, eps)
    want = torch.nn.functional.rms_norm(t64(x), (n,), t64(g), eps).numpy()
    np.testing.assert_allclose(y, want, rtol=1e-13)
    # unit gain and eps = 0: every output row has RMS exactly 1
    y1 = O.rmsnorm_ij_j(x, np.ones(n), 0.0)
    np.testing.assert_allclose(np.sqrt((y1 ** 2).mean(1)), 1.0, rtol=1e-14)
    # scale equivariance at eps = 0
    np.testing.assert_allclose(O.rmsnorm_ij_j(-3.0 * x, g, 0.0), -O.rmsnorm_ij_j(x, g, 0.0), rtol=1e-13)
    # eps sits inside the root, added to the mean (not the sum)
    xs = np.full((1, 4), 2.0)
    np.testing.assert_allclose(O.rmsnorm_ij_j(xs, np.ones(4), 5.0), 2.0 / 3.0, rtol=1e-15)


def test_rmsnorm_reverse_vs_autograd_and_invariants():
    m, n, eps = 23, 130, 1e-6
    x = RNG.normal(0, 1, (m, n))
    g = RNG.normal(1, 0.02, n)
    dy = RNG.normal(0, 1, (m, n))
    xt, gt = t64(x).requires_grad_(True), t64(g).requires_grad_(True)
    torch.nn.functional.rms_norm(xt, (n,), gt, eps).backward(t64(dy))
    dx, dg = O.rmsnorm_ij_j_reverse(x, g, dy, eps)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-11, atol=1e-14)
    np.testing.assert_allclose(dg, gt.grad.numpy(), rtol=1e-11, atol=1e-14)
    # dx is orthogonal to x when eps = 0
    dx0, _ = O.rmsnorm_ij_j_reverse(x, g, dy, 0.0)
    np.testing.assert_allclose((dx0 * x).sum(1), 0.0, atol=1e-12)
    # dg is the column sum of dy * (y / g)
    y = O.rmsnorm_ij_j(x, g, eps)
    np.testing.assert_allclose(dg, (dy * y / g).sum(0), rtol=1e-11, atol=1e-13)
    # blends
    dxi, dgi = RNG.normal(0, 1, (m, n)), RNG.normal(0, 1, n)
    dx2, dg2 = O.rmsnorm_ij_j_reverse(x, g, dy, eps, dxi, dgi, 1.0)
    np.testing.assert_allclose(dx2, dx + dxi, rtol=1e-13, atol=1e-15)
    np.testing.assert_allclose(dg2, dg + dgi, rtol=1e-13, atol=1e-15)
    # the row-parallel timing variant computes the same thing
    dx3, dg3 = O.rmsnorm_ij_j_reverse_mt(x, g, dy, eps)
    np.testing.assert_allclose(dx3, dx, rtol=1e-15)
    np.testing.assert_allclose(dg3, dg, rtol=1e-12, atol=1e-14)
