"""Operands of more than 2^32 elements: every offset in the kernels must be 64-bit. The CPU oracle
checks windows of the result (the start, both sides of element 2^31 and of element 2^32, the end);
properties that hold for every row, and exact or float64 torch expressions, cover the rest."""
import pytest
import torch

import gpu_lib as G
import oracle_lib as O

pytestmark = pytest.mark.gpu

F16 = torch.float16
N_COLS = 2048
M_ROWS = (1 << 21) + 5  # M_ROWS * N_COLS = 2^32 + 10240 elements


def _free():
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def _row_windows(m, n):
    """Rows at the start, around elements 2^31 and 2^32, and at the end."""
    rows = set(range(3))
    for e in (1 << 31, 1 << 32):
        r = e // n
        rows.update(x for x in range(r - 2, r + 3) if 0 <= x < m)
    rows.update(range(m - 3, m))
    return torch.tensor(sorted(rows), device="cuda")


def _flat_windows(n, width=4096):
    spans = [(0, width), ((1 << 31) - width, (1 << 31) + width), ((1 << 32) - width, min(n, (1 << 32) + width)),
             (n - width, n)]
    return [(a, b) for (a, b) in spans if 0 <= a < b <= n]


def test_elementwise_beyond_32_bit_offsets():
    n = (1 << 32) + 4099
    G.say(f"addition r16 n={n}")
    a = torch.randn(n, device="cuda", dtype=F16)
    b = torch.randn(n, device="cuda", dtype=F16)
    c = torch.empty_like(a)
    G.addition(a, b, c)
    torch.cuda.synchronize()
    for (lo, hi) in _flat_windows(n):
        G.compare(c[lo:hi], O.addition(G.host(a[lo:hi]), G.host(b[lo:hi])), F16, f"addition window [{lo},{hi})")
    # both add in fp32 and round once to r16: torch's own addition must agree bit for bit
    assert torch.equal(c, a + b)
    G.say(f"fill r16 n={n}")
    G.fill(c, 0.25)
    torch.cuda.synchronize()
    assert bool((c == 0.25).all())
    del a, b, c
    _free()


def test_softmax_beyond_32_bit_offsets():
    m, n = M_ROWS, N_COLS
    G.say(f"softmax forward r16 [{m},{n}]")
    x = torch.randn(m, n, device="cuda", dtype=F16).mul_(2)
    y = torch.empty_like(x)
    G.softmax(x, y)
    torch.cuda.synchronize()
    rows = _row_windows(m, n)
    G.compare(y[rows], O.softmax_ij_j(G.host(x[rows])), F16, "softmax windows", **G.softmax_tol(F16))
    sums = torch.zeros(m, device="cuda", dtype=torch.float32)
    step = 1 << 18
    for r in range(0, m, step):
        sums[r:r + step] = y[r:r + step].float().sum(dim=1)
    assert bool(torch.isfinite(sums).all()) and float((sums - 1).abs().max()) < 5e-3, "rows must sum to one"
    assert bool((y >= 0).all())

    G.say(f"softmax reverse r16 [{m},{n}]")
    dy = x  # the input has served its purpose: reuse it as the upstream gradient
    dx = torch.empty_like(y)
    G.softmax_reverse(y, dy, dx)
    torch.cuda.synchronize()
    yh, dyh = G.host(y[rows]), G.host(dy[rows])
    G.compare(dx[rows], O.softmax_ij_j_reverse(yh, dyh), F16, "softmax reverse windows",
              scale=G.softmax_reverse_scale(yh, dyh))
    # sum_j dx_ij = dot_i * (1 - sum_j y_ij): zero up to the r16 rounding of y and dx
    worst = 0.0
    for r in range(0, m, step):
        worst = max(worst, float(dx[r:r + step].float().sum(dim=1).abs().max()))
    assert worst < 5e-2, f"rows of dx must sum to zero, worst {worst}"
    del x, y, dy, dx
    _free()


def test_rmsnorm_beyond_32_bit_offsets():
    m, n, eps = M_ROWS, N_COLS, 1e-6
    G.say(f"rmsnorm forward r16 [{m},{n}]")
    x = torch.randn(m, n, device="cuda", dtype=F16)
    g = (1 + 0.02 * torch.randn(n, device="cuda")).to(F16)
    y = torch.empty_like(x)
    G.rmsnorm(x, g, y, eps)
    torch.cuda.synchronize()
    rows = _row_windows(m, n)
    G.compare(y[rows], O.rmsnorm_ij_j(G.host(x[rows]), G.host(g), eps), F16, "rmsnorm windows")
    # every row of y / gain has mean square one
    step = 1 << 18
    worst = 0.0
    for r in range(0, m, step):
        ms = (y[r:r + step].float() / g.float()).pow(2).mean(dim=1)
        worst = max(worst, float((ms - 1).abs().max()))
    assert worst < 1e-2, f"mean square of y / gain, worst deviation {worst}"

    G.say(f"rmsnorm reverse r16 [{m},{n}]")
    del y
    dy = torch.randn(m, n, device="cuda", dtype=F16)
    dx = torch.empty_like(x)
    dg = torch.empty_like(g)
    scratch, _ = G.rmsnorm_scratch(F16, m, n)
    G.rmsnorm_reverse(x, g, dy, dx, dg, scratch.t, eps)
    torch.cuda.synchronize()
    scratch.check("rmsnorm reverse scratch")
    xh, gh, dyh = G.host(x[rows]), G.host(g), G.host(dy[rows])
    ref_dx, _ = O.rmsnorm_ij_j_reverse(xh, gh, dyh, eps)
    sdx, _ = G.rmsnorm_reverse_scales(xh, gh, dyh, eps)
    G.compare(dx[rows], ref_dx, F16, "rmsnorm reverse windows", scale=sdx)
    # the gain gradient sums over all rows: float64 torch expression of sum_i dy * x * r, in slabs
    ref_dg = torch.zeros(n, device="cuda", dtype=torch.float64)
    slab = 1 << 16
    for r in range(0, m, slab):
        xs, ds = x[r:r + slab].double(), dy[r:r + slab].double()
        inv = torch.rsqrt(xs.pow(2).mean(dim=1, keepdim=True) + eps)
        ref_dg += (ds * xs * inv).sum(dim=0)
    G.compare(dg, ref_dg.cpu().numpy(), F16, "rmsnorm gain gradient", rowwise=False)
    del x, dy, dx, scratch
    _free()


def test_matrix_kernels_beyond_32_bit_offsets():
    m, n = 65536 + 8, 65536 + 24  # 2^32 + 2^21 + ... elements, both sides pack-aligned
    G.say(f"permutate r16 [{m},{n}]")
    x = torch.randn(m, n, device="cuda", dtype=F16)
    t = torch.empty(n, m, device="cuda", dtype=F16)
    G.permutate(x, t)
    torch.cuda.synchronize()
    assert torch.equal(t, x.t())
    del t
    _free()

    G.say(f"reduce_ij_i / reduce_ij_j r16 [{m},{n}]")
    si = torch.empty(m, device="cuda", dtype=F16)
    sj = torch.empty(n, device="cuda", dtype=F16)
    G.matrix_op("reduce_ij_i", x, si, 0.0, m, n)
    G.matrix_op("reduce_ij_j", x, sj, 0.0, m, n)
    torch.cuda.synchronize()
    ref_i = torch.zeros(m, device="cuda", dtype=torch.float64)
    ref_j = torch.zeros(n, device="cuda", dtype=torch.float64)
    slab = 4096
    for r in range(0, m, slab):
        xs = x[r:r + slab].double()
        ref_i[r:r + slab] = xs.sum(dim=1)
        ref_j += xs.sum(dim=0)
    # against the float64 torch sums: relative to max(|sum|, RMS of all the sums)
    G.compare(si, ref_i.cpu().numpy(), F16, "row sums", rowwise=False)
    G.compare(sj, ref_j.cpu().numpy(), F16, "column sums", rowwise=False)
    rows = _row_windows(m, n)
    G.compare(si[rows], O.reduce_ij_i(G.host(x[rows])), F16, "row sums, oracle windows", rowwise=False)

    G.say(f"broadcast_i_ij / broadcast_j_ij r16 [{m},{n}]")
    G.matrix_op("broadcast_i_ij", si, x, 0.0, m, n)
    torch.cuda.synchronize()
    assert torch.equal(x, si[:, None].expand(m, n))
    G.matrix_op("broadcast_j_ij", sj, x, 0.0, m, n)
    torch.cuda.synchronize()
    assert torch.equal(x, sj[None, :].expand(m, n))
    del x
    _free()
