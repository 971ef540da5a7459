"""GPU parity of the transpose and the matrix products, through the C-ABI, against the fp64
oracle. The products are compared with a tolerance relative to the size of the summed terms
(|alpha| * sum_j |a_ij b_jk| + |beta c_ik|): r32 1e-5, r16 2e-3, r64 1e-12 of that."""
import numpy as np
import pytest
import torch

import gpu_lib as G
import oracle_lib as O

pytestmark = pytest.mark.gpu

DTYPES = [torch.float16, torch.float32, torch.float64]
IDS = ["r16", "r32", "r64"]


def rng(seed):
    return np.random.default_rng(seed)


# rows x cols: single element, vectors, tiles exactly, one past a tile, ragged both ways,
# odd sizes that force the peeled (memory-aligned) paths on one side or both, with whole tiles and cut ones
TRANSPOSE_SHAPES = [(1, 1), (1, 7), (7, 1), (3, 2), (64, 64), (128, 128), (65, 64), (64, 65), (129, 257),
                    (32, 1000), (1000, 32), (8, 4096), (50257, 3), (100, 104), (104, 100), (1027, 513),
                    (520, 777), (1030, 66), (2049, 130)]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shift", [0, 1])
def test_permutate_forward_and_blend(dtype, shift):
    r = rng(31)
    for (rows, cols) in TRANSPOSE_SHAPES:
        for alpha in (0.0, 1.0, -0.5):
            G.say(f"permutate dtype={dtype} shape=({rows},{cols}) alpha={alpha} shift={shift}")
            src = G.dev(r.normal(0, 1, (rows, cols)), dtype, shift)
            dst = G.dev(r.normal(0, 1, (cols, rows)), dtype, shift)
            before = G.host(dst.t).copy()
            G.permutate(src.t, dst.t, alpha)
            ref = O.permutate_ij_ji(G.host(src.t), before if alpha else None, alpha)
            if alpha == 0.0:
                assert np.array_equal(G.host(dst.t).astype(np.float64), ref), "transpose must move bits unchanged"
            else:
                G.compare(dst.t, ref, dtype, f"permutate ({rows},{cols}) alpha {alpha}", rowwise=False,
                          scale=np.abs(G.host(src.t).T.astype(np.float64)) + abs(alpha) * np.abs(before.astype(np.float64)))
            dst.check("permutate dst")
            src.check("permutate src")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_permutate_narrow_matrices(dtype):
    """A short side of up to 64 (160 when fields are gathered into records): records to fields and back through the chunked kernel; chunk
    boundaries (8192 / n records for r32), cut packs on either side, shifted bases, blend."""
    r = rng(38)
    for n in (1, 2, 3, 4, 5, 7, 8, 12, 16, 31, 33, 63, 64, 65, 130, 160, 161):
        for (m, shifts) in ((1, (0, 0)), (6, (1, 0)), (1000, (0, 0)), (8193, (0, 1)), (40003, (1, 3))):
            for (rows, cols) in ((m, n), (n, m)):
                for alpha in (0.0, -0.5):
                    G.say(f"permutate narrow dtype={dtype} shape=({rows},{cols}) alpha={alpha} shifts={shifts}")
                    src = G.dev(r.normal(0, 1, (rows, cols)), dtype, shifts[0])
                    dst = G.dev(r.normal(0, 1, (cols, rows)), dtype, shifts[1])
                    before = G.host(dst.t).copy()
                    G.permutate(src.t, dst.t, alpha)
                    ref = O.permutate_ij_ji(G.host(src.t), before if alpha else None, alpha)
                    if alpha == 0.0:
                        assert np.array_equal(G.host(dst.t).astype(np.float64), ref), "transpose must move bits unchanged"
                    else:
                        G.compare(dst.t, ref, dtype, f"permutate ({rows},{cols}) alpha {alpha}", rowwise=False,
                                  scale=np.abs(G.host(src.t).T.astype(np.float64)) + abs(alpha) * np.abs(before.astype(np.float64)))
                    dst.check("permutate dst")
                    src.check("permutate src")


def test_permutate_mixed_alignment_and_empty():
    f32 = torch.float32
    r = rng(32)
    for (s_shift, d_shift) in ((0, 1), (1, 0), (3, 2)):
        G.say(f"permutate r32 (96,200) shifts {s_shift},{d_shift}")
        src = G.dev(r.normal(0, 1, (96, 200)), f32, s_shift)
        dst = G.Guarded((200, 96), f32, d_shift)
        G.permutate(src.t, dst.t)
        assert torch.equal(dst.t, src.t.t())
        dst.check("permutate")
    G.say("permutate with an empty dimension")
    src, dst = G.Guarded((0, 5), f32), G.Guarded((5, 0), f32)
    G.permutate(src.t, dst.t)
    torch.cuda.synchronize()
    dst.check("empty permutate")


def test_permutate_involution_at_size():
    # a large ragged matrix: transposing twice returns every bit (size-independent property)
    G.say("permutate r16 (8191, 4104) twice")
    x = torch.randn(8191, 4104, device="cuda").to(torch.float16)
    y = torch.empty(4104, 8191, dtype=torch.float16, device="cuda")
    z = torch.empty_like(x)
    G.permutate(x, y)
    G.permutate(y, z)
    assert torch.equal(y, x.t())
    assert torch.equal(z, x)


GEMM_SHAPES = [(1, 1, 1), (3, 2, 2), (2, 3, 4), (5, 7, 3), (1, 64, 9), (9, 64, 1), (33, 1, 17), (64, 64, 64),
               (129, 255, 65), (256, 1024, 96), (7, 4099, 5),
               # products with a vector run on the row / column sum kernels
               (1, 5000, 300), (300, 5000, 1), (129, 1, 255), (1, 4099, 7), (2000, 33, 1), (1, 777, 1)]
FORMS = [("ij_jk_ik", False, False), ("ij_kj_ik", False, True), ("ji_jk_ik", True, False)]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_inner_product_every_operand_form(dtype):
    r = rng(33)
    with G.BlasStream() as bs:
        for (m, n, k) in GEMM_SHAPES:
            for form, ta, tb in FORMS:
                for alpha, beta in ((1.0, 0.0), (0.5, 1.0), (-2.0, -0.25)):
                    G.say(f"inner_product_{form} dtype={dtype} m,n,k=({m},{n},{k}) alpha={alpha} beta={beta}")
                    a = G.dev(r.normal(0, 1, (n, m) if ta else (m, n)), dtype)
                    b = G.dev(r.normal(0, 1, (k, n) if tb else (n, k)), dtype)
                    c = G.dev(r.normal(0, 1, (m, k)), dtype)
                    before = G.host(c.t).copy()
                    bs.inner_product(form, a.t, b.t, alpha, c.t, beta, m, n, k)
                    ref, scale = O.inner_product(G.host(a.t), G.host(b.t), alpha, before if beta else None, beta,
                                                 ta=ta, tb=tb, with_scale=True)
                    G.compare(c.t, ref, dtype, f"inner_product_{form} ({m},{n},{k}) {alpha},{beta}", rowwise=False,
                              scale=scale)
                    c.check("inner product c")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_inner_product_of_few_outputs_and_a_long_contraction(dtype):
    """C of at most 8 x 8 over a contraction of thousands to a million: the kernel that keeps every sum
    in registers and splits the contraction over workgroups, every operand form, shifted bases,
    contraction lengths around whole steps."""
    r = rng(39)
    with G.BlasStream() as bs:
        for (m, n, k) in [(4, 8192, 4), (2, 8193, 3), (8, 8200, 8), (5, 100003, 7), (3, 20011, 2), (4, 1 << 20, 4),
                          (8, 300007, 5), (2, 9000, 2), (7, 8191, 7)]:
            for form, ta, tb in FORMS:
                for (alpha, beta, shift) in ((1.0, 0.0, 0), (-0.5, 0.75, 1)):
                    G.say(f"few outputs {form} dtype={dtype} m,n,k=({m},{n},{k}) alpha={alpha} beta={beta} shift={shift}")
                    a = G.dev(r.normal(0, 1, (n, m) if ta else (m, n)), dtype, shift)
                    b = G.dev(r.normal(0, 1, (k, n) if tb else (n, k)), dtype, shift)
                    c = G.dev(r.normal(0, 1, (m, k)), dtype, shift)
                    before = G.host(c.t).copy()
                    bs.inner_product(form, a.t, b.t, alpha, c.t, beta, m, n, k)
                    ref, scale = O.inner_product(G.host(a.t), G.host(b.t), alpha, before if beta else None, beta,
                                                 ta=ta, tb=tb, with_scale=True)
                    G.compare(c.t, ref, dtype, f"few outputs {form} ({m},{n},{k}) {alpha},{beta}", rowwise=False,
                              scale=scale)
                    for gd in (a, b, c):
                        gd.check("few outputs")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_inner_product_of_many_rows_through_a_tiny_matrix(dtype):
    """C[m, k] with n, k <= 8 and a thousand rows or more: the kernel that gives a thread one row, every
    operand form, row lengths on and off the 4- and 8-element packs, shifted bases, and row counts
    whose last rows cannot be read as whole packs."""
    r = rng(41)
    with G.BlasStream() as bs:
        for (m, n, k) in [(4096, 4, 4), (1024, 8, 8), (70001, 3, 4), (50003, 4, 3), (33333, 2, 2), (20001, 5, 8),
                          (20001, 8, 5), (10007, 7, 7), (9001, 2, 8), (9001, 8, 2), (1025, 6, 3), (1 << 18, 4, 4)]:
            for form, ta, tb in FORMS:
                for (alpha, beta, shift) in ((1.0, 0.0, 0), (-0.5, 0.75, 1)):
                    G.say(f"tiny matrix {form} dtype={dtype} m,n,k=({m},{n},{k}) alpha={alpha} beta={beta} shift={shift}")
                    a = G.dev(r.normal(0, 1, (n, m) if ta else (m, n)), dtype, shift)
                    b = G.dev(r.normal(0, 1, (k, n) if tb else (n, k)), dtype, shift)
                    c = G.dev(r.normal(0, 1, (m, k)), dtype, shift)
                    before = G.host(c.t).copy()
                    bs.inner_product(form, a.t, b.t, alpha, c.t, beta, m, n, k)
                    ref, scale = O.inner_product(G.host(a.t), G.host(b.t), alpha, before if beta else None, beta,
                                                 ta=ta, tb=tb, with_scale=True)
                    G.compare(c.t, ref, dtype, f"tiny matrix {form} ({m},{n},{k}) {alpha},{beta}", rowwise=False,
                              scale=scale)
                    for gd in (a, b, c):
                        gd.check("tiny matrix")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_inner_product_of_many_rows_with_a_few_vectors(dtype):
    """C[m, k] with 2 <= k <= 8 and thousands of rows of any length: the kernel that walks four rows at a
    time against the k vectors, for B stored as the vectors and as their transpose, row lengths around
    whole packs and around the group widths, shifted bases, row counts that leave a group short of rows."""
    r = rng(43)
    with G.BlasStream() as bs:
        for (m, n, k) in [(4096, 512, 2), (2048, 1024, 8), (1025, 2049, 3), (70001, 33, 5), (300001, 9, 8),
                          (5003, 4099, 7), (1024, 2048, 4), (40002, 64, 8), (9001, 257, 6), (3001, 1000, 2),
                          (1027, 8200, 8)]:
            for form, ta, tb in FORMS[:2]:
                for (alpha, beta, shift) in ((1.0, 0.0, 0), (-0.5, 0.75, 1)):
                    G.say(f"few vectors {form} dtype={dtype} m,n,k=({m},{n},{k}) alpha={alpha} beta={beta} shift={shift}")
                    a = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
                    b = G.dev(r.normal(0, 1, (k, n) if tb else (n, k)), dtype, shift)
                    c = G.dev(r.normal(0, 1, (m, k)), dtype, shift)
                    before = G.host(c.t).copy()
                    bs.inner_product(form, a.t, b.t, alpha, c.t, beta, m, n, k)
                    ref, scale = O.inner_product(G.host(a.t), G.host(b.t), alpha, before if beta else None, beta,
                                                 ta=ta, tb=tb, with_scale=True)
                    G.compare(c.t, ref, dtype, f"few vectors {form} ({m},{n},{k}) {alpha},{beta}", rowwise=False,
                              scale=scale)
                    for gd in (a, b, c):
                        gd.check("few vectors")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_inner_product_of_long_rows_from_a_few_terms(dtype):
    """C[m, k] over a contraction of 2 to 8 with rows of C longer than that: the kernel that keeps a
    piece of B in registers and writes a pack column of four rows a thread, for B stored either way,
    row lengths around whole packs, shifted bases, row counts that leave the last threads short of
    rows; the last shape has rows long enough to stay with the library."""
    r = rng(47)
    with G.BlasStream() as bs:
        for (m, n, k) in [(1 << 15, 8, 64), (70001, 3, 33), (300001, 5, 9), (40000, 4, 100), (20001, 7, 127),
                          (16385, 2, 128), (150001, 8, 17), (262147, 6, 12), (5003, 7, 4099)]:
            for form, ta, tb in FORMS[:2]:
                for (alpha, beta, shift) in ((1.0, 0.0, 0), (-0.5, 0.75, 1)):
                    G.say(f"few terms {form} dtype={dtype} m,n,k=({m},{n},{k}) alpha={alpha} beta={beta} shift={shift}")
                    a = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
                    b = G.dev(r.normal(0, 1, (k, n) if tb else (n, k)), dtype, shift)
                    c = G.dev(r.normal(0, 1, (m, k)), dtype, shift)
                    before = G.host(c.t).copy()
                    bs.inner_product(form, a.t, b.t, alpha, c.t, beta, m, n, k)
                    ref, scale = O.inner_product(G.host(a.t), G.host(b.t), alpha, before if beta else None, beta,
                                                 ta=ta, tb=tb, with_scale=True)
                    G.compare(c.t, ref, dtype, f"few terms {form} ({m},{n},{k}) {alpha},{beta}", rowwise=False,
                              scale=scale)
                    for gd in (a, b, c):
                        gd.check("few terms")


def test_inner_product_reference_example():
    # src/examples/experimental.zig:19-34,51-62: z = x.y, then the reverse with a seed of ones
    f32 = torch.float32
    x = G.dev(np.array([[1, 2], [3, 4], [5, 6]]), f32)
    y = G.dev(np.array([[1, 2], [3, 4]]), f32)
    z, gz = G.Guarded((3, 2), f32), G.dev(np.ones((3, 2)), f32)
    gx, gy = G.dev(np.zeros((3, 2)), f32), G.dev(np.zeros((2, 2)), f32)
    with G.BlasStream() as bs:
        G.say("experimental example: ij,jk->ik and its two reverse products")
        bs.inner_product("ij_jk_ik", x.t, y.t, 1.0, z.t, 0.0, 3, 2, 2)
        bs.inner_product("ij_kj_ik", gz.t, y.t, 1.0, gx.t, 1.0, 3, 2, 2)   # dx = G(z).T(y)
        bs.inner_product("ji_jk_ik", x.t, gz.t, 1.0, gy.t, 1.0, 2, 3, 2)   # dy = T(x).G(z)
    assert z.t.tolist() == [[7, 10], [15, 22], [23, 34]]
    assert gx.t.tolist() == [[3, 7]] * 3
    assert gy.t.tolist() == [[9, 9], [12, 12]]


def test_inner_product_at_size_is_linear_in_its_operands():
    # 4096^3 in r16: (A1 + A2).B against A1.B + A2.B accumulated with beta = 1; both sides come
    # from the launcher, the tolerance is r16 output rounding on sums of 4096 products
    n = 4096
    G.say("inner_product r16 4096^3 linearity")
    a1 = (torch.randn(n, n, device="cuda") * 0.25).to(torch.float16)
    a2 = (torch.randn(n, n, device="cuda") * 0.25).to(torch.float16)
    s = (a1.float() + a2.float())
    exact = s.to(torch.float16).float() == s            # rows of A1 + A2 that r16 holds exactly
    a2 = torch.where(exact, a2, torch.zeros_like(a2))   # keep the sum exact everywhere
    asum = (a1.float() + a2.float()).to(torch.float16)
    b = (torch.randn(n, n, device="cuda") * 0.25).to(torch.float16)
    c_sum = torch.empty(n, n, dtype=torch.float16, device="cuda")
    c_acc = torch.empty_like(c_sum)
    with G.BlasStream() as bs:
        bs.inner_product("ij_jk_ik", asum, b, 1.0, c_sum, 0.0, n, n, n)
        bs.inner_product("ij_jk_ik", a1, b, 1.0, c_acc, 0.0, n, n, n)
        bs.inner_product("ij_jk_ik", a2, b, 1.0, c_acc, 1.0, n, n, n)
    scale = float((a1.float().abs().mean() + a2.float().abs().mean()) * b.float().abs().mean() * n)
    err = (c_sum.float() - c_acc.float()).abs().max().item()
    assert err <= 4e-3 * scale, (err, scale)


def test_r16_vector_products_keep_subnormal_inputs():
    """The r16 matrix-vector product multiplies packed halves (v_dot2_f32_f16); subnormal matrix
    entries must still count: against a large vector they add up to ordinary values."""
    f16 = torch.float16
    m, n = 64, 4096
    a = np.full((m, n), 3e-6)  # below the smallest normal r16 value (6.1e-5)
    a[:, ::7] = 2.5e-7
    A = G.dev(a, f16)
    v, u = G.dev(np.full((n, 1), 2048.0), f16), G.dev(np.full((1, m), 2048.0), f16)
    av, ua = G.Guarded((m, 1), f16), G.Guarded((1, n), f16)
    with G.BlasStream() as stream:
        G.say("A.v and u.A with subnormal r16 entries")
        stream.inner_product("ij_jk_ik", A.t, v.t, 1.0, av.t, 0.0, m, n, 1)
        stream.inner_product("ij_jk_ik", u.t, A.t, 1.0, ua.t, 0.0, 1, m, n)
    ref_av, ref_ua = O.inner_product(G.host(A.t), G.host(v.t)), O.inner_product(G.host(u.t), G.host(A.t))
    assert float(ref_av.min()) > 20.0 and float(ref_ua.min()) > 0.03
    G.compare(av.t, ref_av, f16, "A.v with subnormal entries", rowwise=False)
    G.compare(ua.t, ref_ua, f16, "u.A with subnormal entries", rowwise=False)
    for gd in (A, v, u, av, ua):
        gd.check("subnormal products")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_sums_and_dot_products_of_few_long_rows(dtype):
    """The sum or dot product of whole tensors: one to a few very long rows. On a stream made by
    mpInitStream the rows are cut into segments through the stream's workspace (two launches,
    fixed order); results must match the oracle like any other row sum."""
    r = rng(36)
    with G.BlasStream() as stream:
        for (m, n, shift) in [(1, 100003, 0), (3, 250000, 0), (8, 70001, 1), (1, 1 << 21, 0), (40, 40000, 0)]:
            for alpha in (0.0, -0.5):
                G.say(f"long rows dtype={dtype} shape=({m},{n}) shift={shift} alpha={alpha}")
                x = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
                v = G.dev(r.normal(0, 1, (n, 1)), dtype, shift)
                s = G.dev(r.normal(0, 1, m), dtype)
                d = G.dev(r.normal(0, 1, (m, 1)), dtype)
                bs, bd = G.host(s.t).copy(), G.host(d.t).copy()
                stream.matrix_op("reduce_ij_i", x.t, s.t, alpha, m, n)
                stream.inner_product("ij_jk_ik", x.t, v.t, 1.0, d.t, alpha, m, n, 1)
                xh = G.host(x.t)
                mag = np.abs(xh.astype(np.float64)).sum(axis=1) + abs(alpha) * np.abs(bs.astype(np.float64))
                G.compare(s.t, O.reduce_ij_i(xh, bs if alpha else None, alpha), dtype, f"row sums ({m},{n})",
                          rowwise=False, scale=mag)
                ref, scale = O.inner_product(xh, G.host(v.t), 1.0, bd if alpha else None, alpha, with_scale=True)
                G.compare(d.t, ref, dtype, f"A.v ({m},{n})", rowwise=False, scale=scale)
                # one row against a matrix stored [k, n]: k dot products of length n
                k = 3
                b = G.dev(r.normal(0, 1, (k, n)), dtype)
                c = G.dev(r.normal(0, 1, (1, k)), dtype)
                bc = G.host(c.t).copy()
                row = G.dev(G.host(x.t)[:1].astype(np.float64), dtype)
                stream.inner_product("ij_kj_ik", row.t, b.t, 0.5, c.t, alpha, 1, n, k)
                ref, scale = O.inner_product(G.host(row.t), G.host(b.t), 0.5, bc if alpha else None, alpha, tb=True,
                                             with_scale=True)
                G.compare(c.t, ref, dtype, f"a.B^T ({k},{n})", rowwise=False, scale=scale)
                for gd in (x, v, s, d, b, c, row):
                    gd.check("long rows")
        # the column sums of a few long rows (the sum of a handful of vectors) and u.A
        for (m, n, shift) in [(1, 100003, 0), (2, 5000, 1), (3, 250000, 0), (8, 70001, 1), (40, 40000, 0), (65, 3000, 0),
                              (256, 2049, 0), (257, 2049, 1), (5, 511, 0)]:
            for alpha in (0.0, -0.5):
                G.say(f"short matrix dtype={dtype} shape=({m},{n}) shift={shift} alpha={alpha}")
                x = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
                xh = G.host(x.t)
                sj = G.dev(r.normal(0, 1, n), dtype, shift)
                bj = G.host(sj.t).copy()
                stream.matrix_op("reduce_ij_j", x.t, sj.t, alpha, m, n)
                ax = np.abs(xh.astype(np.float64))
                G.compare(sj.t, O.reduce_ij_j(xh, bj if alpha else None, alpha), dtype, f"column sums ({m},{n})",
                          rowwise=False, scale=ax.sum(axis=0) + abs(alpha) * np.abs(bj.astype(np.float64)))
                u, e = G.dev(r.normal(0, 1, (1, m)), dtype), G.dev(r.normal(0, 1, (1, n)), dtype, shift)
                be = G.host(e.t).copy()
                stream.inner_product("ij_jk_ik", u.t, x.t, -0.5, e.t, alpha, 1, m, n)
                ref, scale = O.inner_product(G.host(u.t), xh, -0.5, be if alpha else None, alpha, with_scale=True)
                G.compare(e.t, ref, dtype, f"u.A ({m},{n})", rowwise=False, scale=scale)
                for gd in (x, sj, u, e):
                    gd.check("short matrix")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_sums_and_products_of_tall_narrow_matrices(dtype):
    """Rows of one element up to a few packs: row sums and A.v take a thread (or 2, 4, 8 lanes) per
    row, column sums and v.A as many lanes per row as the row has packs, broadcasts the flat kernel."""
    r = rng(37)
    with G.BlasStream() as stream:
        for (m, n, shift) in [(70001, 1, 0), (50003, 2, 1), (40001, 3, 0), (30011, 4, 0), (30011, 5, 1), (20001, 7, 0),
                              (20000, 8, 0), (9001, 9, 1), (9001, 15, 0), (8192, 16, 0), (7001, 17, 0), (5003, 31, 1),
                              (4096, 32, 0), (5003, 33, 0), (3001, 63, 0), (3001, 65, 1), (2049, 127, 0), (3, 5, 0)]:
            for alpha in (0.0, 0.75):
                G.say(f"narrow dtype={dtype} shape=({m},{n}) shift={shift} alpha={alpha}")
                x = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
                xh = G.host(x.t)
                si, sj = G.dev(r.normal(0, 1, m), dtype), G.dev(r.normal(0, 1, n), dtype, shift)
                bi, bj = G.host(si.t).copy(), G.host(sj.t).copy()
                stream.matrix_op("reduce_ij_i", x.t, si.t, alpha, m, n)
                stream.matrix_op("reduce_ij_j", x.t, sj.t, alpha, m, n)
                ax = np.abs(xh.astype(np.float64))
                G.compare(si.t, O.reduce_ij_i(xh, bi if alpha else None, alpha), dtype, f"row sums ({m},{n})",
                          rowwise=False, scale=ax.sum(axis=1) + abs(alpha) * np.abs(bi.astype(np.float64)))
                G.compare(sj.t, O.reduce_ij_j(xh, bj if alpha else None, alpha), dtype, f"column sums ({m},{n})",
                          rowwise=False, scale=ax.sum(axis=0) + abs(alpha) * np.abs(bj.astype(np.float64)))
                # A.v: one dot product a row; u.A: the rows weighted and summed
                v, d = G.dev(r.normal(0, 1, (n, 1)), dtype, shift), G.dev(r.normal(0, 1, (m, 1)), dtype)
                u, e = G.dev(r.normal(0, 1, (1, m)), dtype), G.dev(r.normal(0, 1, (1, n)), dtype, shift)
                bd, be = G.host(d.t).copy(), G.host(e.t).copy()
                stream.inner_product("ij_jk_ik", x.t, v.t, 1.0, d.t, alpha, m, n, 1)
                stream.inner_product("ij_jk_ik", u.t, x.t, -0.5, e.t, alpha, 1, m, n)
                ref, scale = O.inner_product(xh, G.host(v.t), 1.0, bd if alpha else None, alpha, with_scale=True)
                G.compare(d.t, ref, dtype, f"A.v ({m},{n})", rowwise=False, scale=scale)
                ref, scale = O.inner_product(G.host(u.t), xh, -0.5, be if alpha else None, alpha, with_scale=True)
                G.compare(e.t, ref, dtype, f"u.A ({m},{n})", rowwise=False, scale=scale)
                # the product of a column and a row vector, into a copy of the matrix
                col, rowv = G.dev(r.normal(0, 1, (m, 1)), dtype), G.dev(r.normal(0, 1, (1, n)), dtype, shift)
                c = G.dev(xh.astype(np.float64), dtype, shift)
                stream.inner_product("ij_jk_ik", col.t, rowv.t, 0.5, c.t, alpha, m, 1, n)
                ref, scale = O.inner_product(G.host(col.t), G.host(rowv.t), 0.5, xh if alpha else None, alpha, with_scale=True)
                G.compare(c.t, ref, dtype, f"outer product ({m},{n})", rowwise=False, scale=scale)
                for gd in (col, rowv, c):
                    gd.check("outer product")
                # the reverses: both broadcasts into a copy of the matrix
                for op, vec in (("broadcast_i_ij", si), ("broadcast_j_ij", sj)):
                    y = G.dev(xh.astype(np.float64), dtype, shift)
                    stream.matrix_op(op, vec.t, y.t, alpha, m, n)
                    ref = getattr(O, op)(G.host(vec.t), m, n, xh if alpha else None, alpha)
                    vh = np.abs(G.host(vec.t).astype(np.float64))
                    G.compare(y.t, ref, dtype, f"{op} ({m},{n})", rowwise=False,
                              scale=(vh[:, None] if op == "broadcast_i_ij" else vh[None, :]) + abs(alpha) * ax)
                    y.check(op)
                for gd in (x, si, sj, v, d, u, e):
                    gd.check("narrow")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_inner_product_on_both_sides_of_every_dispatch_threshold(dtype):
    """The launcher picks between the library's GEMM and four kernels of its own by size thresholds
    (rows from 1024, tensors from 2^21 elements, contractions from 8192, sides of at most 8, rows of
    C of at most 128): the shape just below and just above each of them, for both transposes and a
    blend, must give the same answer whichever kernel takes it."""
    r = rng(53)
    shapes = [
        # tiny map: n, k <= 8 and m >= 1024
        (1023, 8, 8), (1024, 8, 8), (1024, 9, 8), (1024, 8, 9),
        # few terms: 2 <= n <= 8 < k <= 128 and m * k >= 2^21
        (16384, 8, 127), (16384, 8, 128), (16384, 8, 129), (16383, 8, 128), (262144, 2, 8), (262144, 2, 9),
        (262144, 1, 9), (233017, 8, 9), (233018, 9, 9),
        # few dots: 2 <= k <= 8 < n, m >= 1024 and m * n >= 2^21
        (1023, 2051, 8), (1024, 2048, 8), (1024, 2047, 8), (1024, 2048, 9), (2048, 1024, 2), (2048, 1023, 2),
        # small product: m, k <= 8 and n >= 8192
        (8, 8191, 8), (8, 8192, 8), (9, 8192, 8), (8, 8192, 9), (4, 8192, 4), (4, 8191, 4),
    ]
    with G.BlasStream() as bs:
        for (m, n, k) in shapes:
            for form, ta, tb in FORMS:
                for (alpha, beta) in ((1.0, 0.0), (-0.5, 0.75)):
                    G.say(f"threshold {form} dtype={dtype} m,n,k=({m},{n},{k}) alpha={alpha} beta={beta}")
                    a = G.dev(r.normal(0, 1, (n, m) if ta else (m, n)), dtype)
                    b = G.dev(r.normal(0, 1, (k, n) if tb else (n, k)), dtype)
                    c = G.dev(r.normal(0, 1, (m, k)), dtype)
                    before = G.host(c.t).copy()
                    bs.inner_product(form, a.t, b.t, alpha, c.t, beta, m, n, k)
                    ref, scale = O.inner_product(G.host(a.t), G.host(b.t), alpha, before if beta else None, beta,
                                                 ta=ta, tb=tb, with_scale=True)
                    G.compare(c.t, ref, dtype, f"threshold {form} ({m},{n},{k}) {alpha},{beta}", rowwise=False,
                              scale=scale)
                    for gd in (a, b, c):
                        gd.check("threshold")
