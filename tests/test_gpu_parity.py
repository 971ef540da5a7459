"""GPU parity: every launcher, through the C-ABI, against the fp64 CPU oracle on the same
seeded inputs, at sizes the oracle finishes in seconds. Buffers carry canaries; ragged,
unaligned, aliased, empty and masked inputs are covered, and the softmax / RMSNorm launchers
are driven through each row regime."""
import numpy as np
import pytest
import torch

import gpu_lib as G
import oracle_lib as O

pytestmark = pytest.mark.gpu

DTYPES = [torch.float16, torch.float32, torch.float64]
IDS = ["r16", "r32", "r64"]
REGIMES = [0, 1, 2, 3, 4, 5, 6, 7, 8, 9]  # auto, G = 64..1024, stream, cluster (softmax fwd), G = 16, 32 (softmax)


@pytest.fixture(autouse=True)
def _auto_regime():
    G.set_regime(0)
    G.set_cluster_tuning()
    G.set_cluster_deep()
    yield
    G.set_regime(0)
    G.set_cluster_tuning()
    G.set_cluster_deep()
    torch.cuda.synchronize()


def rng(seed):
    return np.random.default_rng(seed)


# ------------------------------------------------------------------ elementwise

EW_SIZES = [0, 1, 3, 8, 255, 1024, 4099, (1 << 20) + 5]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shift", [0, 1])
def test_add_hadamard_and_reverse(dtype, shift):
    r = rng(10)
    for n in EW_SIZES:
        G.say(f"add/hadamard dtype={dtype} n={n} shift={shift}")
        a, b = G.dev(r.normal(0, 1, n), dtype, shift), G.dev(r.normal(0, 1, n), dtype, shift)
        c = G.Guarded((n,), dtype, shift)
        G.addition(a.t, b.t, c.t)
        G.compare(c.t, O.addition(G.host(a.t), G.host(b.t)), dtype, f"addition n={n}", rowwise=False)
        G.hadamard(a.t, b.t, c.t)
        G.compare(c.t, O.hadamard(G.host(a.t), G.host(b.t)), dtype, f"hadamard n={n}", rowwise=False)
        c0 = G.dev(r.normal(0, 1, n), dtype, shift)
        before = G.host(c0.t).copy()
        G.hadamard_reverse(a.t, b.t, c0.t)
        G.compare(c0.t, O.hadamard_reverse(G.host(a.t), G.host(b.t), before), dtype,
                  f"hadamard_reverse n={n}", rowwise=False)
        for g in (a, b, c, c0):
            g.check(f"elementwise n={n}")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shift", [0, 1])
def test_remaining_elementwise_launchers(dtype, shift):
    r = rng(14)
    npdt = G.NP_OF[dtype]
    for n in [0, 1, 5, 1000, 65537]:
        G.say(f"sub/negate/relu/step/dilate/translate/fill/sequence/copy dtype={dtype} n={n} shift={shift}")
        x = r.normal(0, 1, n)
        x[: min(n, 2)] = [0.0, -0.0][: min(n, 2)]
        a, b = G.dev(x, dtype, shift), G.dev(r.normal(0, 1, n), dtype, shift)
        ha, hb = G.host(a.t), G.host(b.t)
        c = G.Guarded((n,), dtype, shift)
        G.subtraction(a.t, b.t, c.t)
        G.compare(c.t, O.subtraction(ha, hb), dtype, f"subtraction n={n}", rowwise=False)
        for stem, ref in (("negate", O.negate), ("relu", O.relu), ("stepwise", O.stepwise), ("copy", O.copy)):
            G.unary(stem, a.t, c.t)
            G.compare(c.t, ref(ha), dtype, f"{stem} n={n}", rowwise=False, rtol=0.0 if stem != "relu" else None)
        acc = G.dev(r.normal(0, 1, n), dtype, shift)
        before = G.host(acc.t).copy()
        G.relu_reverse(a.t, acc.t, b.t)
        G.compare(acc.t, O.relu_reverse(ha, hb, before), dtype, f"relu_reverse n={n}", rowwise=False)
        G.scalar_op("dilate", a.t, 0.3, c.t)
        G.compare(c.t, O.dilate(ha, 0.3), dtype, f"dilate n={n}", rowwise=False)
        G.scalar_op("translate", a.t, -1.7, c.t)
        G.compare(c.t, O.translate(ha, -1.7), dtype, f"translate n={n}", rowwise=False)
        acc = G.dev(r.normal(0, 1, n), dtype, shift)
        before = G.host(acc.t).copy()
        G.scalar_op("dilate_reverse", a.t, 0.3, acc.t)
        G.compare(acc.t, O.dilate_reverse(ha, 0.3, before), dtype, f"dilate_reverse n={n}", rowwise=False)
        G.fill(c.t, 1.0)
        assert bool((c.t == 1).all())
        G.fill(c.t, 0.1)
        G.compare(c.t, O.fill(npdt, 0.1, n), dtype, f"fill n={n}", rowwise=False, rtol=0.0)
        G.sequence(c.t, 0.5, 0.25)
        G.compare(c.t, O.sequence(npdt, 0.5, 0.25, n), dtype, f"sequence n={n}", rowwise=False)
        for g in (a, b, c, acc):
            g.check(f"remaining elementwise n={n}")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_elementwise_operand_layouts(dtype):
    """Operands at the start of a cache line, all at the same other place of one (the first elements
    are peeled off), 16-byte aligned at different places, and at places that differ by single
    elements (packs that start anywhere); lengths around the peeled head and the pack width."""
    r = rng(24)
    for n in (1, 5, 17, 31, 32, 33, 40, 63, 64, 65, 71, 100, 1000, 4099, 70001):
        for shifts in ((0, 0, 0), (1, 1, 1), (5, 5, 5), (4, 4, 4), (8, 8, 8), (4, 8, 0), (1, 0, 0), (0, 0, 3), (1, 2, 3), (31, 31, 31)):
            G.say(f"elementwise layouts dtype={dtype} n={n} shifts={shifts}")
            a = G.dev(r.normal(0, 1, n), dtype, shifts[0])
            b = G.dev(r.normal(0, 1, n), dtype, shifts[1])
            c = G.Guarded((n,), dtype, shifts[2])
            G.addition(a.t, b.t, c.t)
            assert torch.equal(c.t, a.t + b.t), f"addition n={n} shifts={shifts}"
            G.hadamard(a.t, b.t, c.t)
            assert torch.equal(c.t, a.t * b.t), f"hadamard n={n} shifts={shifts}"
            for gd in (a, b, c):
                gd.check("elementwise layouts")


def test_reference_example_all_ones_through_relu_add():
    # src/examples/subgraphs.zig:34-45: x = w1 = w2 = 1; z4 = relu(relu(x + w1) + w2) == 3
    f32 = torch.float32
    n = 32
    x, w1, w2 = (G.Guarded((n,), f32) for _ in range(3))
    for t in (x, w1, w2):
        G.fill(t.t, 1.0)
    z1, z2, z3, z4 = (G.Guarded((n,), f32) for _ in range(4))
    G.say("subgraphs example: relu(add) twice")
    G.addition(x.t, w1.t, z1.t)
    G.unary("relu", z1.t, z2.t)
    G.addition(z2.t, w2.t, z3.t)
    G.unary("relu", z3.t, z4.t)
    assert bool((z4.t == 3).all())
    # reverse: seed dz4 = 1 (graph.zig:116), then relu_reverse / in-place addition as the ops do
    grads = {k: G.dev(np.zeros(n), f32) for k in ("z4", "z3", "z2", "z1", "x", "w1", "w2")}
    G.fill(grads["z4"].t, 1.0)
    G.relu_reverse(z3.t, grads["z3"].t, grads["z4"].t)
    G.addition(grads["z3"].t, grads["z2"].t, grads["z2"].t)
    G.addition(grads["z3"].t, grads["w2"].t, grads["w2"].t)
    G.relu_reverse(z1.t, grads["z1"].t, grads["z2"].t)
    G.addition(grads["z1"].t, grads["x"].t, grads["x"].t)
    G.addition(grads["z1"].t, grads["w1"].t, grads["w1"].t)
    for k in ("x", "w1", "w2"):
        assert bool((grads[k].t == 1).all()), k


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_addition_in_place_as_the_reference_reverse_calls_it(dtype):
    # src/ops/addition.zig:67-73: gx = gz + gx with the output aliasing the second input
    r = rng(11)
    n = 70001
    gz, gx = G.dev(r.normal(0, 1, n), dtype), G.dev(r.normal(0, 1, n), dtype)
    want = O.addition(G.host(gz.t), G.host(gx.t))
    G.say(f"addition in place dtype={dtype}")
    G.addition(gz.t, gx.t, gx.t)
    G.compare(gx.t, want, dtype, "in-place addition", rowwise=False)
    gx.check("in-place addition")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shift", [0, 1])
def test_selu_forward_and_reverse(dtype, shift):
    r = rng(12)
    for n in EW_SIZES:
        G.say(f"selu dtype={dtype} n={n} shift={shift}")
        x = r.uniform(-9, 9, n)
        x[: min(n, 6)] = [0.0, -0.0, 1e-4, -1e-4, -0.25, -0.2500001][: min(n, 6)]
        a = G.dev(x, dtype, shift)
        b = G.Guarded((n,), dtype, shift)
        G.selu(a.t, b.t)
        G.compare(b.t, O.selu(G.host(a.t)), dtype, f"selu n={n}", rowwise=False)
        gb, ga = G.dev(r.normal(0, 1, n), dtype, shift), G.dev(r.normal(0, 1, n), dtype, shift)
        before = G.host(ga.t).copy()
        G.selu_reverse(a.t, ga.t, gb.t)
        G.compare(ga.t, O.selu_reverse(G.host(a.t), G.host(gb.t), before), dtype,
                  f"selu_reverse n={n}", rowwise=False)
        for g in (a, b, ga, gb):
            g.check(f"selu n={n}")


def test_selu_relative_accuracy_near_zero_r32():
    # the expm1 branch must keep relative accuracy where exp(x)-1 cancels
    x = -np.logspace(-8, 0.5, 4000)
    a = G.dev(x, torch.float32)
    b = G.Guarded(a.t.shape, torch.float32)
    G.say("selu near zero r32")
    G.selu(a.t, b.t)
    ref = O.selu(G.host(a.t))
    got = b.t.double().cpu().numpy()
    assert np.max(np.abs(got - ref) / np.abs(ref)) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shift", [0, 1])
def test_fused_chain_forward_and_reverse(dtype, shift):
    r = rng(13)
    for n in EW_SIZES:
        G.say(f"fused dtype={dtype} n={n} shift={shift}")
        ins = [G.dev(r.uniform(-2, 2, n), dtype, shift) for _ in range(4)]
        de = G.dev(r.normal(0, 1, n), dtype, shift)
        e = G.Guarded((n,), dtype, shift)
        G.fused(*[g.t for g in ins], e.t)
        hin = [G.host(g.t) for g in ins]
        G.compare(e.t, O.fused_selu_hadamard_add_add(*hin), dtype, f"fused fwd n={n}", rowwise=False)
        outs = [G.Guarded((n,), dtype, shift) for _ in range(4)]
        G.fused_reverse(*[g.t for g in ins], de.t, *[g.t for g in outs], alpha=0.0)
        refs = O.fused_selu_hadamard_add_add_reverse(*hin, G.host(de.t))
        for name, g, ref in zip("abcd", outs, refs):
            G.compare(g.t, ref, dtype, f"fused rev d{name} n={n}", rowwise=False)
        if n:
            assert torch.equal(outs[0].t, outs[1].t) and torch.equal(outs[2].t, outs[3].t)
        # accumulate mode: out = val + alpha*old
        olds = [G.dev(r.normal(0, 1, n), dtype, shift) for _ in range(4)]
        hold = tuple(G.host(g.t).copy() for g in olds)
        G.fused_reverse(*[g.t for g in ins], de.t, *[g.t for g in olds], alpha=1.0)
        refs = O.fused_selu_hadamard_add_add_reverse(*hin, G.host(de.t), hold, alpha=1.0)
        for name, g, ref in zip("abcd", olds, refs):
            G.compare(g.t, ref, dtype, f"fused rev accumulate d{name} n={n}", rowwise=False)
        for g in ins + outs + olds + [de, e]:
            g.check(f"fused n={n}")


# ------------------------------------------------------------------ generated chains

def _chain_cases():
    from metaphor_amd import chaingen
    return [(c["name"], c["expr"]) for c in chaingen.load_chains()]


@pytest.mark.parametrize("name,expr", _chain_cases(), ids=[c[0] for c in _chain_cases()])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_generated_chain_launchers(name, expr, dtype):
    """Every chain of chains.json through the C-ABI against fp64 torch (forward and autograd) on
    the same rounded inputs; alpha = 0 overwrites, alpha = 1 accumulates."""
    from metaphor_amd import chaingen
    from test_chaingen import _torch_eval
    root, k = chaingen.parse(expr)
    r = rng(16)
    for n in [1, 7, 1000, 65539]:
        G.say(f"chain {name} dtype={dtype} n={n}")
        xs = [G.dev(r.uniform(-2, 2, n), dtype) for _ in range(k)]
        up = G.dev(r.normal(0, 1, n), dtype)
        ts = [torch.from_numpy(G.host(x.t).astype(np.float64)).requires_grad_(True) for x in xs]
        ref = _torch_eval(root, ts)
        ref.backward(torch.from_numpy(G.host(up.t).astype(np.float64)))
        out = G.Guarded((n,), dtype)
        G._call(name, dtype, *[x.t.data_ptr() for x in xs], out.t.data_ptr(), n)
        G.compare(out.t, ref.detach().numpy(), dtype, f"{name} forward n={n}", rowwise=False)
        for alpha in (0.0, 1.0):
            gs = [G.dev(r.normal(0, 1, n), dtype) for _ in range(k)]
            olds = [G.host(g.t).astype(np.float64) for g in gs]
            G._call(name + "_reverse", dtype, *[x.t.data_ptr() for x in xs], up.t.data_ptr(),
                    *[g.t.data_ptr() for g in gs], float(alpha), n)
            for i in range(k):
                want = ts[i].grad.numpy() + alpha * olds[i]
                # terms of a sum may cancel (sub, repeated leaves): scale by their size
                scale = np.abs(ts[i].grad.numpy()) + alpha * np.abs(olds[i])
                G.compare(gs[i].t, want, dtype, f"{name} reverse g{i} alpha={alpha} n={n}", rowwise=False, scale=scale)
                gs[i].check(name)
        out.check(name)


# ------------------------------------------------------------------ reduce / broadcast

MATRIX_SHAPES = [(1, 1), (3, 2), (2, 2), (7, 5), (33, 64), (64, 1000), (5, 1027), (300, 4096), (2, 50257),
                 (4100, 36), (2, 20000)]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shift", [0, 1])
def test_reduce_and_broadcast(dtype, shift):
    r = rng(15)
    for (m, n) in MATRIX_SHAPES:
        for alpha in (0.0, 1.0):
            G.say(f"reduce/broadcast dtype={dtype} shape=({m},{n}) alpha={alpha} shift={shift}")
            src = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            hs = G.host(src.t)
            for stem, ref_fn, k in (("reduce_ij_i", O.reduce_ij_i, m), ("reduce_ij_j", O.reduce_ij_j, n)):
                dst = G.dev(r.normal(0, 1, k), dtype, shift)
                before = G.host(dst.t).copy()
                G.matrix_op(stem, src.t, dst.t, alpha, m, n)
                ref = ref_fn(hs, before if alpha else None, alpha)
                scale = np.abs(hs.astype(np.float64)).sum(axis=1 if stem == "reduce_ij_i" else 0)
                G.compare(dst.t, ref, dtype, f"{stem} ({m},{n}) alpha {alpha}", rowwise=False, scale=scale)
                dst.check(stem)
            for stem, ref_fn, k in (("broadcast_i_ij", O.broadcast_i_ij, m), ("broadcast_j_ij", O.broadcast_j_ij, n)):
                vec = G.dev(r.normal(0, 1, k), dtype, shift)
                dst = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
                before = G.host(dst.t).copy()
                G.matrix_op(stem, vec.t, dst.t, alpha, m, n)
                ref = ref_fn(G.host(vec.t), m, n, before if alpha else None, alpha)
                G.compare(dst.t, ref, dtype, f"{stem} ({m},{n}) alpha {alpha}")
                dst.check(stem)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_column_sums_with_workspace(dtype):
    """Tall matrices: the rows are split into chunks whose partial rows a second kernel adds up."""
    r = rng(16)
    used = 0
    for (m, n) in [(3, 2), (700, 8), (5000, 64), (4097, 1024), (20000, 40), (1500, 1027), (33, 64)]:
        for alpha in (0.0, 1.0):
            for scratch in ("auto", None):
                G.say(f"reduce_ij_j_scratch dtype={dtype} shape=({m},{n}) alpha={alpha} scratch={scratch}")
                src = G.dev(r.normal(0, 1, (m, n)), dtype)
                dst = G.dev(r.normal(0, 1, n), dtype)
                before = G.host(dst.t).copy()
                used += bool(G.reduce_ij_j_scratch(src.t, dst.t, alpha, m, n, scratch))
                ref = O.reduce_ij_j(G.host(src.t), before if alpha else None, alpha)
                scale = np.abs(G.host(src.t).astype(np.float64)).sum(axis=0) + abs(alpha) * np.abs(before.astype(np.float64))
                G.compare(dst.t, ref, dtype, f"reduce_ij_j_scratch ({m},{n}) alpha {alpha}", rowwise=False, scale=scale)
                dst.check("column sums")
    assert used > 0, "no shape took the two-stage path"


def test_column_sums_without_a_workspace_say_so_at_most_once(capfd):
    """launch_reduce_ij_j through a bare stream context has no workspace to split a tall, narrow
    matrix through: the result is the same, and the library says what that costs once a process."""
    r = rng(18)
    f32 = torch.float32
    notes = 0
    for (m, n) in [(60000, 8), (90001, 12)]:
        G.say(f"reduce_ij_j through a bare context shape=({m},{n})")
        src, dst = G.dev(r.normal(0, 1, (m, n)), f32), G.Guarded((n,), f32)
        capfd.readouterr()
        G.matrix_op("reduce_ij_j", src.t, dst.t, 0.0, m, n)
        torch.cuda.synchronize()
        notes += capfd.readouterr().err.count("given no workspace")
        ref = O.reduce_ij_j(G.host(src.t), None, 0.0)
        G.compare(dst.t, ref, f32, f"reduce_ij_j bare ({m},{n})", rowwise=False,
                  scale=np.abs(G.host(src.t).astype(np.float64)).sum(axis=0))
        dst.check("column sums")
    assert notes <= 1, "the note about the missing workspace was printed more than once"


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_column_sums_on_a_library_stream(dtype):
    """launch_reduce_ij_j has the reference's signature (no workspace): on a stream made by
    mpInitStream it splits tall matrices through the workspace that the stream context owns."""
    r = rng(17)
    with G.BlasStream() as stream:
        for (m, n) in [(3, 2), (5000, 64), (4097, 1024), (20000, 40), (1500, 1027), (70000, 256)]:
            for alpha in (0.0, -0.5):
                G.say(f"reduce_ij_j on a library stream dtype={dtype} shape=({m},{n}) alpha={alpha}")
                src = G.dev(r.normal(0, 1, (m, n)), dtype)
                dst = G.dev(r.normal(0, 1, n), dtype)
                before = G.host(dst.t).copy()
                stream.matrix_op("reduce_ij_j", src.t, dst.t, alpha, m, n)
                ref = O.reduce_ij_j(G.host(src.t), before if alpha else None, alpha)
                scale = np.abs(G.host(src.t).astype(np.float64)).sum(axis=0) + abs(alpha) * np.abs(before.astype(np.float64))
                G.compare(dst.t, ref, dtype, f"reduce_ij_j ({m},{n}) alpha {alpha}", rowwise=False, scale=scale)
                dst.check("column sums")
                src.check("column sums source")


def test_reference_example_reductions():
    # src/examples/experimental.zig:19-34
    f32 = torch.float32
    x = G.dev(np.array([[1, 2], [3, 4], [5, 6]]), f32)
    y = G.dev(np.array([[1, 2], [3, 4]]), f32)
    yi, xj = G.Guarded((2,), f32), G.Guarded((2,), f32)
    G.say("experimental example: reduce ij->i and ij->j")
    G.matrix_op("reduce_ij_i", y.t, yi.t, 0.0, 2, 2)
    G.matrix_op("reduce_ij_j", x.t, xj.t, 0.0, 3, 2)
    assert yi.t.tolist() == [3.0, 7.0] and xj.t.tolist() == [9.0, 12.0]


# ------------------------------------------------------------------ softmax

SOFTMAX_SHAPES = [(1, 1), (3, 7), (5, 64), (4, 65), (1031, 16), (9, 256), (7, 1000), (256, 1024), (6, 2048),
                  (3, 5000), (5, 8192), (2, 20000), (3, 32768), (2, 50257), (3, 65536), (1, 151936), (1030, 33), (2051, 8), (515, 32)]


def _softmax_inputs(r, m, n, dtype, masked):
    x = r.normal(0, 2, (m, n))
    if masked:
        rows, cols = np.indices((m, n))
        x[cols > (rows % max(n, 1))] = -np.inf
    return x


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("regime", REGIMES)
def test_softmax_forward_all_regimes(dtype, regime):
    r = rng(20 + regime)
    G.set_regime(regime)
    for (m, n) in SOFTMAX_SHAPES:
        for masked in (False, True):
            G.say(f"softmax fwd dtype={dtype} regime={regime} shape=({m},{n}) masked={masked}")
            x = G.dev(_softmax_inputs(r, m, n, dtype, masked), dtype)
            y = G.Guarded((m, n), dtype)
            G.softmax(x.t, y.t)
            ref = O.softmax_ij_j(G.host(x.t))
            G.compare(y.t, ref, dtype, f"softmax ({m},{n}) regime {regime}", **G.softmax_tol(dtype))
            if masked:
                assert bool((y.t[torch.isinf(x.t)] == 0).all()), "-inf must map to exactly 0"
            x.check("softmax x")
            y.check("softmax y")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("regime", [0, 6])
def test_softmax_unaligned_bases_and_in_place(dtype, regime):
    r = rng(30)
    G.set_regime(regime)
    for (m, n) in [(5, 100), (3, 1027), (2, 50257), (4, 4096)]:
        for sx, sy in [(1, 1), (1, 0), (3, 2)]:
            G.say(f"softmax unaligned dtype={dtype} regime={regime} shape=({m},{n}) shifts=({sx},{sy})")
            x = G.dev(r.normal(0, 3, (m, n)), dtype, sx)
            y = G.Guarded((m, n), dtype, sy)
            G.softmax(x.t, y.t)
            ref = O.softmax_ij_j(G.host(x.t))
            G.compare(y.t, ref, dtype, f"softmax unaligned ({m},{n})", **G.softmax_tol(dtype))
            x.check("x")
            y.check("y")
        x = G.dev(r.normal(0, 3, (m, n)), dtype)
        ref = O.softmax_ij_j(G.host(x.t))
        G.say(f"softmax in place dtype={dtype} shape=({m},{n})")
        G.softmax(x.t, x.t)
        G.compare(x.t, ref, dtype, f"softmax in place ({m},{n})", **G.softmax_tol(dtype))
        x.check("in place")


CLUSTER = 7


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("packs,spin", [(0, 1 << 22), (64, 1 << 22), (3, 1 << 22), (64, 0), (1000, 2)],
                         ids=["default", "64packs", "3packs", "64packs-nowait", "1000packs-2polls"])
def test_softmax_forward_cluster_path(dtype, packs, spin):
    """Several workgroups per row with the (max, sum) exchange through scratch. A spin limit of 0
    or 2 polls makes most workgroups give up waiting and fold the whole row themselves: every
    kernel still ends and the results stay within tolerance."""
    r = rng(32)
    G.set_regime(CLUSTER)
    G.set_cluster_tuning(packs, spin)
    for (m, n) in [(3, 7), (5, 64), (4, 1000), (6, 2048), (33, 5000), (2, 50257), (2, 151936), (130, 777)]:
        for masked in (False, True):
            for shift in (0, 1):
                G.say(f"softmax cluster dtype={dtype} packs={packs} spin={spin} shape=({m},{n}) masked={masked} shift={shift}")
                x = G.dev(_softmax_inputs(r, m, n, dtype, masked), dtype, shift)
                y = G.Guarded((m, n), dtype, shift)
                G.softmax(x.t, y.t)
                ref = O.softmax_ij_j(G.host(x.t))
                G.compare(y.t, ref, dtype, f"softmax cluster ({m},{n}) packs {packs} spin {spin}",
                          **G.softmax_tol(dtype))
                if masked:
                    assert bool((y.t[torch.isinf(x.t)] == 0).all())
                x.check("x")
                y.check("y")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_forward_results_do_not_depend_on_what_is_left_in_the_cache(dtype):
    """The forward kernels come in two flavours that differ in a cache hint alone: the RMSNorm forward
    loads x, and the softmax forward stores y, so that the tensor stays in the memory-side cache
    for the reverse (tensors up to a size) or streams past it (larger ones). Both flavours of every
    kernel that has them, forced through the test build: the same bits, and within the bound of the
    oracle. Row lengths: one per forward path (one-shot groups, persistent groups, groups of whole
    wavefronts, eight rows a workgroup, rows shared by workgroups)."""
    r = rng(53)
    eps = 1e-6
    try:
        for (m, n) in [(37, 512), (19, 1152), (23, 1280), (9, 4096), (5, 16384), (3, 50257), (2, 151936)]:
            x = G.dev(r.normal(0, 2, (m, n)), dtype)
            g = G.dev(1 + 0.1 * r.normal(0, 1, n), dtype)
            xh, gh = G.host(x.t), G.host(g.t)
            got = {}
            for mode in (0, 1):
                G.set_keep_input(mode)
                G.say(f"cache policy {mode} dtype={dtype} shape=({m},{n})")
                y, z = G.Guarded((m, n), dtype), G.Guarded((m, n), dtype)
                G.rmsnorm(x.t, g.t, y.t, eps)
                G.softmax(x.t, z.t)
                G.compare(y.t, O.rmsnorm_ij_j(xh, gh, eps), dtype, f"rmsnorm policy {mode} ({m},{n})")
                G.compare(z.t, O.softmax_ij_j(xh), dtype, f"softmax policy {mode} ({m},{n})", **G.softmax_tol(dtype))
                y.check("y")
                z.check("z")
                got[mode] = (y.t.clone(), z.t.clone())
            assert torch.equal(got[0][0], got[1][0]), f"rmsnorm ({m},{n}): the two flavours differ"
            assert torch.equal(got[0][1], got[1][1]), f"softmax ({m},{n}): the two flavours differ"
    finally:
        G.set_keep_input(2)


@pytest.mark.parametrize("own", [1, 0], ids=["library-words", "caller-words"])
def test_shared_row_softmax_launch_after_launch(own):
    """The stamped exchange words of the shared-row softmax kernels: launch after launch through one
    workspace with fresh inputs every time (a word left by the launch before must not pass for a
    result), two geometries taking turns through the same workspace, more workspaces than the
    library has regions for, forward and reverse, in the library's own words (the library as
    shipped) and in the caller's workspace (test build), whole outputs against the oracle."""
    r = rng(37)
    f32 = torch.float32
    G.set_cluster_words(own)
    try:
        shapes = [(6, 50257), (3, 151936)]
        big = max(G.row_size("mpSoftmaxScratchBytes", f32, m, n) for m, n in shapes)
        bigr = max(G.row_size("mpSoftmaxReverseScratchBytes", f32, m, n) for m, n in shapes)
        assert big > 0 and bigr > 0
        fs, rs = G.Guarded((big,), torch.uint8), G.Guarded((bigr,), torch.uint8)
        for launch in range(6):
            m, n = shapes[launch % 2]
            x = G.dev(r.normal(0, 3, (m, n)) + launch, f32)
            dy = G.dev(r.normal(0, 1, (m, n)), f32)
            y, dx = G.Guarded((m, n), f32), G.Guarded((m, n), f32)
            G.say(f"shared rows own={own} launch {launch} ({m},{n})")
            G.softmax(x.t, y.t, scratch=fs.t)
            G.softmax_reverse(y.t, dy.t, dx.t, 0.0, scratch=rs.t)
            yh, dyh = G.host(y.t), G.host(dy.t)
            G.compare(y.t, O.softmax_ij_j(G.host(x.t)), f32, f"shared rows launch {launch}", atol=1e-6)
            G.compare(dx.t, O.softmax_ij_j_reverse(yh, dyh), f32, f"shared rows rev launch {launch}",
                      scale=G.softmax_reverse_scale(yh, dyh))
            for b in (y, dx, fs, rs):
                b.check("shared rows")
        # 70 workspaces at different addresses (the table has 64 regions): the ones beyond fall back
        m, n = 2, 50257
        need = G.row_size("mpSoftmaxScratchBytes", f32, m, n)
        pool = torch.zeros(70 * (need + 256), dtype=torch.uint8, device="cuda")
        x = G.dev(r.normal(0, 3, (m, n)), f32)
        ref = O.softmax_ij_j(G.host(x.t))
        for i in range(70):
            y = G.Guarded((m, n), f32)
            ws = pool[i * (need + 256):(i + 1) * (need + 256)]
            G.say(f"shared rows own={own} workspace {i}")
            G.softmax(x.t, y.t, scratch=ws)
            if i % 10 == 0 or i > 60:
                G.compare(y.t, ref, f32, f"shared rows workspace {i}", atol=1e-6)
                y.check("y")
    finally:
        G.set_cluster_words(1)


def test_shared_row_softmax_replayed_from_a_graph_with_fresh_inputs():
    """A captured forward + reverse over shared rows, replayed with other inputs each time: the stamp
    of a launch is read on the device, so a replay is as good as a fresh launch."""
    r = rng(38)
    f32 = torch.float32
    m, n = 5, 50257
    x = torch.empty((m, n), dtype=f32, device="cuda")
    dy = torch.empty((m, n), dtype=f32, device="cuda")
    y, dx = torch.empty_like(x), torch.empty_like(x)
    fs = torch.empty(G.row_size("mpSoftmaxScratchBytes", f32, m, n), dtype=torch.uint8, device="cuda")
    rs = torch.empty(G.row_size("mpSoftmaxReverseScratchBytes", f32, m, n), dtype=torch.uint8, device="cuda")

    def fresh(k):
        x.copy_(torch.from_numpy(r.normal(0, 3, (m, n)) + k).to(f32))
        dy.copy_(torch.from_numpy(r.normal(0, 1, (m, n))).to(f32))

    def sequence():
        G.softmax(x, y, scratch=fs)
        G.softmax_reverse(y, dy, dx, 0.0, scratch=rs)

    fresh(0)
    G.say("shared rows graph: eager")
    sequence()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sequence()
    for k in range(1, 5):
        fresh(k)
        y.fill_(float("nan"))
        dx.fill_(float("nan"))
        torch.cuda.synchronize()
        G.say(f"shared rows graph: replay {k}")
        graph.replay()
        torch.cuda.synchronize()
        yh, dyh = G.host(y), G.host(dy)
        G.compare(y, O.softmax_ij_j(G.host(x)), f32, f"shared rows replay {k}", atol=1e-6)
        G.compare(dx, O.softmax_ij_j_reverse(yh, dyh), f32, f"shared rows rev replay {k}",
                  scale=G.softmax_reverse_scale(yh, dyh))
        if k == 2:  # eager work through the same workspaces between replays
            sequence()
            torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32], ids=["r16", "r32"])
def test_shared_rows_starting_at_every_offset_from_a_128_byte_line(dtype):
    """Rows of 16 bytes more than a multiple of 128: nine consecutive rows start at each of the
    eight pack offsets from a line, and the chunks of a shared row move back by that offset (the
    first workgroup's first lanes idle, the last chunk ends at the row's end). Forward, reverse
    and RMSNorm forward of the library as shipped, whole outputs against the oracle."""
    r = rng(35)
    per_pack = 16 // torch.empty((), dtype=dtype).element_size()
    n = 10001 * per_pack
    m = 9
    for shift in (0, 1):
        G.say(f"line offsets dtype={dtype} ({m},{n}) shift={shift}")
        x = G.dev(r.normal(0, 2, (m, n)), dtype, shift)
        y = G.Guarded((m, n), dtype, shift)
        G.softmax(x.t, y.t)
        G.compare(y.t, O.softmax_ij_j(G.host(x.t)), dtype, f"softmax line offsets shift {shift}", **G.softmax_tol(dtype))
        dy = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
        dx = G.Guarded((m, n), dtype, shift)
        G.softmax_reverse(y.t, dy.t, dx.t, 0.0)
        yh, dyh = G.host(y.t), G.host(dy.t)
        G.compare(dx.t, O.softmax_ij_j_reverse(yh, dyh), dtype, f"softmax rev line offsets shift {shift}",
                  scale=G.softmax_reverse_scale(yh, dyh))
        g = G.dev(r.normal(1, 0.02, n), dtype, shift)
        z = G.Guarded((m, n), dtype, shift)
        G.rmsnorm(x.t, g.t, z.t, 1e-6)
        G.compare(z.t, O.rmsnorm_ij_j(G.host(x.t), G.host(g.t), 1e-6), dtype, f"rmsnorm line offsets shift {shift}")
        for b in (x, y, dy, dx, g, z):
            b.check("line offsets")


def test_softmax_forward_r16_rows_held_at_three_or_five_packs_a_thread():
    """r16 rows of 1152 ... 1792 packs leave a 1024-thread group at two packs a thread partly idle and
    are held at 3, 5 or 7 packs a thread in a narrower group instead (n = 10240, 12288, 9232 with a
    ragged end, and one element off alignment); masked and plain rows against the oracle."""
    r = rng(36)
    dtype = torch.float16
    for (m, n, shift) in [(9, 10240, 0), (9, 12288, 0), (5, 9232, 0), (5, 12290, 1), (3, 14000, 0)]:
        for masked in (False, True):
            G.say(f"softmax r16 odd plan ({m},{n}) shift={shift} masked={masked}")
            x = G.dev(_softmax_inputs(r, m, n, dtype, masked), dtype, shift)
            y = G.Guarded((m, n), dtype, shift)
            G.softmax(x.t, y.t)
            G.compare(y.t, O.softmax_ij_j(G.host(x.t)), dtype, f"softmax r16 odd plan ({m},{n})", **G.softmax_tol(dtype))
            if masked:
                assert bool((y.t[torch.isinf(x.t)] == 0).all())
            x.check("x")
            y.check("y")


def test_softmax_r16_rows_on_half_the_group():
    """r16 rows that would fill a group at two packs a thread to eleven sixteenths or less run on half
    the group at four (forward: n = 1280, 2560, 2816, 5120, 5632), and rows of 513 ... 768 packs stay at
    two packs a thread on 512 threads in the reverse; with a ragged end and one element off alignment;
    forward (masked and plain) and reverse (both blends) against the oracle."""
    r = rng(37)
    dtype = torch.float16
    for (m, n, shift) in [(9, 1280, 0), (9, 2560, 0), (5, 2816, 0), (7, 5120, 0), (5, 5632, 0), (3, 6144, 0),
                          (5, 5121, 0), (5, 5120, 1), (4, 2563, 1), (300, 4608, 0)]:
        for masked in (False, True):
            G.say(f"softmax r16 half group ({m},{n}) shift={shift} masked={masked}")
            x = G.dev(_softmax_inputs(r, m, n, dtype, masked), dtype, shift)
            y = G.Guarded((m, n), dtype, shift)
            G.softmax(x.t, y.t)
            G.compare(y.t, O.softmax_ij_j(G.host(x.t)), dtype, f"softmax r16 half group ({m},{n})", **G.softmax_tol(dtype))
            if masked:
                assert bool((y.t[torch.isinf(x.t)] == 0).all())
            x.check("x")
            y.check("y")
        for alpha in (0.0, 0.5):
            G.say(f"softmax rev r16 half group ({m},{n}) shift={shift} alpha={alpha}")
            yv = G.dev(O.softmax_ij_j(_softmax_inputs(r, m, n, dtype, False)), dtype, shift)
            dy = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            dx = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            before = G.host(dx.t).copy()
            G.softmax_reverse(yv.t, dy.t, dx.t, alpha)
            ref = O.softmax_ij_j_reverse(G.host(yv.t), G.host(dy.t), before if alpha else None, alpha)
            scale = G.softmax_reverse_scale(G.host(yv.t), G.host(dy.t), before if alpha else None, alpha)
            G.compare(dx.t, ref, dtype, f"softmax rev r16 half group ({m},{n}) alpha {alpha}", scale=scale)
            for g in (yv, dy, dx):
                g.check("softmax rev r16 half group")


def test_softmax_long_rows_without_scratch_take_the_two_pass_kernel():
    r = rng(33)
    for (m, n) in [(3, 151936), (4, 50257)]:
        x = G.dev(r.normal(0, 3, (m, n)), torch.float32)
        y = G.Guarded((m, n), torch.float32)
        G.say(f"softmax NULL scratch ({m},{n})")
        G.softmax(x.t, y.t, scratch=None)
        G.compare(y.t, O.softmax_ij_j(G.host(x.t)), torch.float32, f"no scratch ({m},{n})", atol=1e-6)


def test_softmax_vocabulary_spike_rows_r32():
    # the sampling-path input: N(0,3) logits with +12 on one random column per row
    r = rng(31)
    for (m, n) in [(3, 151936), (4, 50257)]:
        x = r.normal(0, 3, (m, n))
        x[np.arange(m), r.integers(0, n, m)] += 12.0
        xd = G.dev(x, torch.float32)
        y = G.Guarded((m, n), torch.float32)
        G.say(f"softmax vocabulary rows ({m},{n})")
        G.softmax(xd.t, y.t)
        G.compare(y.t, O.softmax_ij_j(G.host(xd.t)), torch.float32, f"vocab ({m},{n})", atol=1e-6)
        y.check("vocab")


def test_softmax_all_masked_row_is_nan_like_the_closed_form():
    x = torch.full((2, 128), float("-inf"), device="cuda", dtype=torch.float32)
    x[1, 5] = 0.0
    y = torch.empty_like(x)
    G.say("softmax all -inf row")
    G.softmax(x, y)
    assert bool(torch.isnan(y[0]).all())
    assert float(y[1, 5]) == 1.0 and float(y[1].sum()) == 1.0


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("regime", REGIMES)
def test_softmax_reverse_all_regimes(dtype, regime):
    r = rng(40 + regime)
    G.set_regime(regime)
    for (m, n) in SOFTMAX_SHAPES:
        for alpha in (0.0, 1.0, 0.5):
            if alpha == 0.5 and n > 5000:
                continue
            G.say(f"softmax rev dtype={dtype} regime={regime} shape=({m},{n}) alpha={alpha}")
            xs = _softmax_inputs(r, m, n, dtype, masked=(m % 2 == 0))
            y64 = O.softmax_ij_j(xs)
            y = G.dev(y64, dtype)
            dy = G.dev(r.normal(0, 1, (m, n)), dtype)
            dx = G.dev(r.normal(0, 1, (m, n)), dtype)
            before = G.host(dx.t).copy()
            G.softmax_reverse(y.t, dy.t, dx.t, alpha)
            ref = O.softmax_ij_j_reverse(G.host(y.t), G.host(dy.t), before if alpha else None, alpha)
            scale = G.softmax_reverse_scale(G.host(y.t), G.host(dy.t), before if alpha else None, alpha)
            G.compare(dx.t, ref, dtype, f"softmax rev ({m},{n}) regime {regime} alpha {alpha}", scale=scale)
            for g in (y, dy, dx):
                g.check("softmax rev")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("packs,spin", [(0, 1 << 22), (64, 1 << 22), (3, 1 << 22), (64, 0), (1000, 2)],
                         ids=["default", "64packs", "3packs", "64packs-nowait", "1000packs-2polls"])
def test_softmax_reverse_cluster_path(dtype, packs, spin):
    """Several workgroups per row exchanging their parts of dot(y, dy) through scratch; with a
    poll limit of 0 or 2 most workgroups give up waiting and read the whole row themselves."""
    r = rng(44)
    G.set_regime(CLUSTER)
    G.set_cluster_tuning(packs, spin)
    for (m, n) in [(3, 7), (5, 64), (4, 1000), (6, 2048), (33, 5000), (2, 50257), (2, 151936), (130, 777)]:
        for alpha in (0.0, 1.0):
            for shift in (0, 1):
                G.say(f"softmax rev cluster dtype={dtype} packs={packs} spin={spin} shape=({m},{n}) alpha={alpha} shift={shift}")
                y = G.dev(O.softmax_ij_j(_softmax_inputs(r, m, n, dtype, masked=(m % 2 == 0))), dtype, shift)
                dy = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
                dx = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
                before = G.host(dx.t).copy()
                G.softmax_reverse(y.t, dy.t, dx.t, alpha)
                ref = O.softmax_ij_j_reverse(G.host(y.t), G.host(dy.t), before if alpha else None, alpha)
                scale = G.softmax_reverse_scale(G.host(y.t), G.host(dy.t), before if alpha else None, alpha)
                G.compare(dx.t, ref, dtype, f"softmax rev cluster ({m},{n}) packs {packs} spin {spin}", scale=scale)
                for g in (y, dy, dx):
                    g.check("softmax rev cluster")


def test_softmax_reverse_long_rows_in_place_and_without_scratch():
    # dx written over dy, and a NULL workspace: both must leave the shared-row path
    r = rng(45)
    f32 = torch.float32
    for (m, n) in [(3, 151936), (4, 50257)]:
        y = G.dev(O.softmax_ij_j(r.normal(0, 3, (m, n))), f32)
        dy = G.dev(r.normal(0, 1, (m, n)), f32)
        ref = O.softmax_ij_j_reverse(G.host(y.t), G.host(dy.t))
        scale = G.softmax_reverse_scale(G.host(y.t), G.host(dy.t))
        dx = G.Guarded((m, n), f32)
        G.say(f"softmax rev NULL scratch ({m},{n})")
        G.softmax_reverse(y.t, dy.t, dx.t, 0.0, scratch=None)
        G.compare(dx.t, ref, f32, f"softmax rev no scratch ({m},{n})", scale=scale)
        G.say(f"softmax rev in place ({m},{n})")
        G.softmax_reverse(y.t, dy.t, dy.t, 0.0)
        G.compare(dy.t, ref, f32, f"softmax rev in place ({m},{n})", scale=scale)
        dy.check("in place")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_softmax_reverse_unaligned(dtype):
    r = rng(41)
    for (m, n) in [(5, 100), (3, 1027), (2, 50257)]:
        for shifts in [(1, 1, 1), (1, 0, 2)]:
            G.say(f"softmax rev unaligned dtype={dtype} shape=({m},{n}) shifts={shifts}")
            y = G.dev(O.softmax_ij_j(r.normal(0, 2, (m, n))), dtype, shifts[0])
            dy = G.dev(r.normal(0, 1, (m, n)), dtype, shifts[1])
            dx = G.Guarded((m, n), dtype, shifts[2])
            G.softmax_reverse(y.t, dy.t, dx.t, 0.0)
            ref = O.softmax_ij_j_reverse(G.host(y.t), G.host(dy.t))
            G.compare(dx.t, ref, dtype, f"softmax rev unaligned ({m},{n})",
                      scale=G.softmax_reverse_scale(G.host(y.t), G.host(dy.t)))
            dx.check("dx")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_softmax_short_rows_any_length_and_alignment(dtype):
    """Rows of one element up to sixteen packs and a little beyond: 1 ... 16 lanes a row, packs
    from the row's first element, cut packs in pieces; every length, bases shifted apart, in
    place, with the reverse's alpha blend, and row counts that leave part of a wavefront dead."""
    r = rng(43)
    lengths = list(range(1, 36)) + [40, 47, 48, 56, 63, 64, 65, 72, 96, 100, 120, 127, 128, 129, 136]
    for n in lengths:
        for (m, shifts) in [(1001, (0, 0, 0)), (77, (1, 3, 2)), (3, (2, 2, 2))]:
            G.say(f"softmax short dtype={dtype} shape=({m},{n}) shifts={shifts}")
            x = G.dev(r.normal(0, 3, (m, n)), dtype, shifts[0])
            y = G.Guarded((m, n), dtype, shifts[1])
            G.softmax(x.t, y.t)
            xh = G.host(x.t)
            G.compare(y.t, O.softmax_ij_j(xh), dtype, f"softmax short ({m},{n})", **G.softmax_tol(dtype))
            x.check("x")
            y.check("y")
            dy = G.dev(r.normal(0, 1, (m, n)), dtype, shifts[2])
            yh, dyh = G.host(y.t), G.host(dy.t)
            for alpha in (0.0, -0.5):
                dx = G.dev(r.normal(0, 1, (m, n)), dtype, shifts[0])
                before = G.host(dx.t).copy()
                G.softmax_reverse(y.t, dy.t, dx.t, alpha)
                ref = O.softmax_ij_j_reverse(yh, dyh, before if alpha else None, alpha)
                G.compare(dx.t, ref, dtype, f"softmax short reverse ({m},{n}) alpha={alpha}",
                          scale=G.softmax_reverse_scale(yh, dyh, before if alpha else None, alpha))
                dx.check("dx")
            G.softmax(x.t, x.t)
            G.compare(x.t, O.softmax_ij_j(xh), dtype, f"softmax short in place ({m},{n})", **G.softmax_tol(dtype))
            x.check("in place")


# ------------------------------------------------------------------ RMSNorm

NORM_SHAPES = [(1, 1), (3, 7), (17, 64), (1031, 16), (259, 128), (33, 256), (64, 4096), (5, 1000), (300, 1024), (3, 50257),
               (2, 70001), (1025, 128), (40, 8192), (5, 16384), (3, 32768), (2, 300000), (2051, 8), (515, 32)]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("regime", REGIMES)
def test_rmsnorm_forward_all_regimes(dtype, regime):
    r = rng(50 + regime)
    G.set_regime(regime)
    eps = 1e-6
    for (m, n) in NORM_SHAPES:
        G.say(f"rmsnorm fwd dtype={dtype} regime={regime} shape=({m},{n})")
        x = G.dev(r.normal(0, 1, (m, n)), dtype)
        g = G.dev(r.normal(1, 0.02, n), dtype)
        y = G.Guarded((m, n), dtype)
        G.rmsnorm(x.t, g.t, y.t, eps)
        G.compare(y.t, O.rmsnorm_ij_j(G.host(x.t), G.host(g.t), eps), dtype, f"rmsnorm ({m},{n}) regime {regime}")
        y.check("rmsnorm y")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("regime", [0, 6])
def test_rmsnorm_forward_unaligned_and_in_place(dtype, regime):
    r = rng(51)
    eps = 1e-6
    G.set_regime(regime)
    for (m, n) in [(5, 100), (3, 1027), (2, 50257), (4, 4096)]:
        for sx, sg, sy in [(1, 0, 1), (1, 1, 0), (0, 1, 0)]:
            G.say(f"rmsnorm unaligned dtype={dtype} shape=({m},{n}) shifts=({sx},{sg},{sy})")
            x = G.dev(r.normal(0, 1, (m, n)), dtype, sx)
            g = G.dev(r.normal(1, 0.02, n), dtype, sg)
            y = G.Guarded((m, n), dtype, sy)
            G.rmsnorm(x.t, g.t, y.t, eps)
            G.compare(y.t, O.rmsnorm_ij_j(G.host(x.t), G.host(g.t), eps), dtype, f"rmsnorm unaligned ({m},{n})")
            y.check("y")
        x = G.dev(r.normal(0, 1, (m, n)), dtype)
        g = G.dev(r.normal(1, 0.02, n), dtype)
        ref = O.rmsnorm_ij_j(G.host(x.t), G.host(g.t), eps)
        G.rmsnorm(x.t, g.t, x.t, eps)
        G.compare(x.t, ref, dtype, f"rmsnorm in place ({m},{n})")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_rmsnorm_forward_rows_on_two_to_five_wavefronts(dtype):
    """Aligned rows that would leave a power-of-two group more than an eighth idle (r16 n = 1152, 1280,
    2560, 5120; r32 n = 576, 640, 1280): groups of two to five wavefronts, three to eight rows a
    persistent workgroup. Row counts around the rows a workgroup holds, and in place."""
    r = rng(68)
    per_pack = 16 // torch.empty((), dtype=dtype).element_size()
    for packs in (129, 144, 160, 223, 257, 300, 320, 447, 520, 640):
        n = packs * per_pack
        for m in (1, 7, 37, 2100):
            G.say(f"rmsnorm fwd wavefront groups dtype={dtype} ({m},{n})")
            x = G.dev(r.normal(0, 1, (m, n)), dtype)
            g = G.dev(r.normal(1, 0.02, n), dtype)
            y = G.Guarded((m, n), dtype)
            G.rmsnorm(x.t, g.t, y.t, 1e-6)
            ref = O.rmsnorm_ij_j(G.host(x.t), G.host(g.t), 1e-6)
            G.compare(y.t, ref, dtype, f"rmsnorm fwd wavefront groups ({m},{n})")
            G.rmsnorm(x.t, g.t, x.t, 1e-6)
            G.compare(x.t, ref, dtype, f"rmsnorm fwd wavefront groups in place ({m},{n})")
            for b in (x, g, y):
                b.check("rmsnorm fwd wavefront groups")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("packs,spin", [(0, 1 << 22), (64, 1 << 22), (3, 1 << 22), (64, 0), (1000, 2)],
                         ids=["default", "64packs", "3packs", "64packs-nowait", "1000packs-2polls"])
def test_rmsnorm_forward_cluster_path(dtype, packs, spin):
    """Several workgroups per row exchanging their parts of sum x^2 through scratch; with a poll
    limit of 0 or 2 most workgroups give up waiting and read the whole row themselves."""
    r = rng(52)
    G.set_regime(CLUSTER)
    G.set_cluster_tuning(packs, spin)
    eps = 1e-6
    for (m, n) in [(3, 7), (5, 64), (4, 1000), (6, 2048), (33, 5000), (2, 50257), (2, 151936), (130, 777)]:
        for shift in (0, 1):
            G.say(f"rmsnorm cluster dtype={dtype} packs={packs} spin={spin} shape=({m},{n}) shift={shift}")
            x = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            g = G.dev(r.normal(1, 0.02, n), dtype, shift)
            y = G.Guarded((m, n), dtype, shift)
            G.rmsnorm(x.t, g.t, y.t, eps)
            G.compare(y.t, O.rmsnorm_ij_j(G.host(x.t), G.host(g.t), eps), dtype,
                      f"rmsnorm cluster ({m},{n}) packs {packs} spin {spin}")
            for b in (x, g, y):
                b.check("rmsnorm cluster")


def test_rmsnorm_long_rows_in_place_and_without_scratch():
    r = rng(53)
    f32 = torch.float32
    for (m, n) in [(3, 151936), (4, 50257)]:
        x = G.dev(r.normal(0, 1, (m, n)), f32)
        g = G.dev(r.normal(1, 0.02, n), f32)
        ref = O.rmsnorm_ij_j(G.host(x.t), G.host(g.t), 1e-6)
        y = G.Guarded((m, n), f32)
        G.say(f"rmsnorm NULL scratch ({m},{n})")
        G.rmsnorm(x.t, g.t, y.t, 1e-6, scratch=None)
        G.compare(y.t, ref, f32, f"rmsnorm no scratch ({m},{n})")
        G.say(f"rmsnorm long rows in place ({m},{n})")
        G.rmsnorm(x.t, g.t, x.t, 1e-6)
        G.compare(x.t, ref, f32, f"rmsnorm in place ({m},{n})")
        x.check("in place")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("regime", REGIMES)
def test_rmsnorm_reverse_all_regimes(dtype, regime):
    r = rng(60 + regime)
    G.set_regime(regime)
    eps = 1e-6
    for (m, n) in NORM_SHAPES:
        for alpha in (0.0, 1.0):
            G.say(f"rmsnorm rev dtype={dtype} regime={regime} shape=({m},{n}) alpha={alpha}")
            x = G.dev(r.normal(0, 1, (m, n)), dtype)
            g = G.dev(r.normal(1, 0.02, n), dtype)
            dy = G.dev(r.normal(0, 1, (m, n)), dtype)
            dx = G.dev(r.normal(0, 1, (m, n)), dtype)
            dg = G.dev(r.normal(0, 1, n), dtype)
            hdx, hdg = G.host(dx.t).copy(), G.host(dg.t).copy()
            scratch, nbytes = G.rmsnorm_scratch(dtype, m, n)
            G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, scratch.t, eps, alpha)
            rdx, rdg = O.rmsnorm_ij_j_reverse(G.host(x.t), G.host(g.t), G.host(dy.t), eps,
                                              hdx if alpha else None, hdg if alpha else None, alpha)
            sdx, sdg = G.rmsnorm_reverse_scales(G.host(x.t), G.host(g.t), G.host(dy.t), eps,
                                                hdx if alpha else None, hdg if alpha else None, alpha)
            G.compare(dx.t, rdx, dtype, f"rmsnorm rev dx ({m},{n}) regime {regime} alpha {alpha}", scale=sdx)
            G.compare(dg.t, rdg, dtype, f"rmsnorm rev dg ({m},{n}) regime {regime} alpha {alpha}",
                      rowwise=False, scale=sdg)
            for gd in (x, g, dy, dx, dg, scratch):
                gd.check("rmsnorm rev")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("packs,spin", [(0, 1 << 22), (64, 1 << 22), (64, 0), (1000, 2)],
                         ids=["default", "64packs", "64packs-nowait", "1000packs-2polls"])
def test_rmsnorm_reverse_cluster_path(dtype, packs, spin):
    """Slices of workgroups sharing every row of the slice, two row sums exchanged per row; with a
    poll limit of 0 or 2 most workgroups give up waiting and read the whole row themselves."""
    r = rng(62)
    G.set_regime(CLUSTER)
    G.set_cluster_tuning(packs, spin)
    eps = 1e-6
    # the last four: rows that are not a whole number of packs, and operands shifted by one element
    for (m, n, shift) in [(3, 8, 0), (5, 64, 0), (4, 1000, 0), (700, 2048, 0), (33, 5000, 0), (2, 50264, 0),
                          (3, 151936, 0), (130, 776, 0), (4, 1001, 0), (3, 50257, 0), (2, 70001, 1), (33, 5000, 1)]:
        for alpha in (0.0, 1.0):
            G.say(f"rmsnorm rev cluster dtype={dtype} packs={packs} spin={spin} shape=({m},{n}) shift={shift} alpha={alpha}")
            x = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            g = G.dev(r.normal(1, 0.02, n), dtype, shift)
            dy = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            dx = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            dg = G.dev(r.normal(0, 1, n), dtype)
            hdx, hdg = G.host(dx.t).copy(), G.host(dg.t).copy()
            scratch, nbytes = G.rmsnorm_scratch(dtype, m, n)
            G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, scratch.t, eps, alpha)
            rdx, rdg = O.rmsnorm_ij_j_reverse(G.host(x.t), G.host(g.t), G.host(dy.t), eps,
                                              hdx if alpha else None, hdg if alpha else None, alpha)
            sdx, sdg = G.rmsnorm_reverse_scales(G.host(x.t), G.host(g.t), G.host(dy.t), eps,
                                                hdx if alpha else None, hdg if alpha else None, alpha)
            G.compare(dx.t, rdx, dtype, f"rmsnorm rev cluster dx ({m},{n}) packs {packs} spin {spin}", scale=sdx)
            G.compare(dg.t, rdg, dtype, f"rmsnorm rev cluster dg ({m},{n}) packs {packs} spin {spin}",
                      rowwise=False, scale=sdg)
            for gd in (x, g, dy, dx, dg, scratch):
                gd.check("rmsnorm rev cluster")


@pytest.mark.parametrize("packs,spin", [(0, 1 << 22), (64, 1 << 22), (64, 0), (1000, 2), (300, 1 << 22)],
                         ids=["default", "64packs", "64packs-nowait", "1000packs-2polls", "300packs"])
def test_rmsnorm_reverse_pipelined_shared_rows(packs, spin):
    """The r32 kernel that publishes the sums of row j + 2 and reads the words of row j + 1 while it
    writes back row j (four register sets, the last wavefront polling), forced onto rows of every
    length: one to more rows than a slice gets through in four iterations, rows of one chunk, rows
    that are not whole packs, operands off their alignment; with a poll limit of 0 or 2 workgroups
    stop waiting and fold whole rows themselves."""
    r = rng(68)
    dtype = torch.float32
    G.set_regime(CLUSTER)
    G.set_cluster_tuning(packs, spin)
    G.set_cluster_deep(1)
    eps = 1e-6
    for (m, n, shift) in [(1, 8, 0), (2, 64, 0), (3, 1000, 0), (4, 2048, 0), (5, 5000, 0), (6, 5000, 0), (7, 5000, 1),
                          (9, 776, 0), (700, 2048, 0), (3000, 1001, 0), (2, 50264, 0), (3, 151936, 0), (3, 50257, 0),
                          (2, 70001, 1), (33, 5000, 1)]:
        for alpha in (0.0, 1.0):
            G.say(f"rmsnorm rev pipelined packs={packs} spin={spin} shape=({m},{n}) shift={shift} alpha={alpha}")
            x = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            g = G.dev(r.normal(1, 0.02, n), dtype, shift)
            dy = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            dx = G.dev(r.normal(0, 1, (m, n)), dtype, shift)
            dg = G.dev(r.normal(0, 1, n), dtype)
            hdx, hdg = G.host(dx.t).copy(), G.host(dg.t).copy()
            scratch, nbytes = G.rmsnorm_scratch(dtype, m, n)
            G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, scratch.t, eps, alpha)
            rdx, rdg = O.rmsnorm_ij_j_reverse(G.host(x.t), G.host(g.t), G.host(dy.t), eps,
                                              hdx if alpha else None, hdg if alpha else None, alpha)
            sdx, sdg = G.rmsnorm_reverse_scales(G.host(x.t), G.host(g.t), G.host(dy.t), eps,
                                                hdx if alpha else None, hdg if alpha else None, alpha)
            G.compare(dx.t, rdx, dtype, f"rmsnorm rev pipelined dx ({m},{n}) packs {packs} spin {spin}", scale=sdx)
            G.compare(dg.t, rdg, dtype, f"rmsnorm rev pipelined dg ({m},{n}) packs {packs} spin {spin}",
                      rowwise=False, scale=sdg)
            for gd in (x, g, dy, dx, dg, scratch):
                gd.check("rmsnorm rev pipelined")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["r32", "r64"])
def test_rmsnorm_reverse_rows_held_at_three_packs_a_thread(dtype):
    """Hidden sizes that are not a power of two: the reverse of the library as shipped holds such a
    row at three packs a thread in a narrower group instead of idling lanes of a wider one (r32
    n = 5120, 6144, 10240, 12288; r64 at half those). Whole problem against the oracle, both blends,
    more rows than one workgroup's share so that the pairing of rows wraps."""
    r = rng(66)
    per_pack = 16 // torch.empty((), dtype=dtype).element_size()
    for packs in (1280, 1536, 2560, 3072):
        n, m = packs * per_pack, 37
        for alpha in (0.0, -0.5):
            G.say(f"rmsnorm rev odd plan dtype={dtype} ({m},{n}) alpha={alpha}")
            x = G.dev(r.normal(0, 1, (m, n)), dtype)
            g = G.dev(r.normal(1, 0.02, n), dtype)
            dy = G.dev(r.normal(0, 1, (m, n)), dtype)
            dx = G.dev(r.normal(0, 1, (m, n)), dtype)
            dg = G.dev(r.normal(0, 1, n), dtype)
            hdx, hdg = G.host(dx.t).copy(), G.host(dg.t).copy()
            scratch, _ = G.rmsnorm_scratch(dtype, m, n)
            G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, scratch.t, 1e-6, alpha)
            xh, gh, dyh = G.host(x.t), G.host(g.t), G.host(dy.t)
            rdx, rdg = O.rmsnorm_ij_j_reverse(xh, gh, dyh, 1e-6, hdx if alpha else None, hdg if alpha else None, alpha)
            sdx, sdg = G.rmsnorm_reverse_scales(xh, gh, dyh, 1e-6, hdx if alpha else None, hdg if alpha else None, alpha)
            G.compare(dx.t, rdx, dtype, f"rmsnorm rev odd plan dx ({m},{n}) alpha {alpha}", scale=sdx)
            G.compare(dg.t, rdg, dtype, f"rmsnorm rev odd plan dg ({m},{n}) alpha {alpha}", rowwise=False, scale=sdg)
            for b in (x, g, dy, dx, dg, scratch):
                b.check("rmsnorm rev odd plan")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_rmsnorm_reverse_rows_on_three_to_six_wavefronts(dtype):
    """Rows of 129 ... 223, 257 ... 447 and (at two packs a thread) 513 ... 896 packs (r16 n = 1280, 2560,
    3072, 5120, 7168; r32 n = 640, 1280, 1536, 2560, 3584): three to seven wavefronts a row, five to two
    rows a workgroup; r32 rows of up to 479 packs run on 128-thread groups at two or four packs a
    thread instead, r16 rows that fill a power-of-two group to eleven sixteenths or more on that
    group. Whole problem against the oracle, both blends, row counts that are not a multiple of the
    rows a workgroup holds, and one that leaves workgroups idle."""
    r = rng(67)
    per_pack = 16 // torch.empty((), dtype=dtype).element_size()
    for packs in (129, 160, 223, 257, 320, 384, 447, 513, 640, 832, 895, 896):
        n = packs * per_pack
        for m in (1, 37, 1000):
            for alpha in (0.0, -0.5):
                G.say(f"rmsnorm rev wavefront groups dtype={dtype} ({m},{n}) alpha={alpha}")
                x = G.dev(r.normal(0, 1, (m, n)), dtype)
                g = G.dev(r.normal(1, 0.02, n), dtype)
                dy = G.dev(r.normal(0, 1, (m, n)), dtype)
                dx = G.dev(r.normal(0, 1, (m, n)), dtype)
                dg = G.dev(r.normal(0, 1, n), dtype)
                hdx, hdg = G.host(dx.t).copy(), G.host(dg.t).copy()
                scratch, _ = G.rmsnorm_scratch(dtype, m, n)
                G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, scratch.t, 1e-6, alpha)
                xh, gh, dyh = G.host(x.t), G.host(g.t), G.host(dy.t)
                rdx, rdg = O.rmsnorm_ij_j_reverse(xh, gh, dyh, 1e-6, hdx if alpha else None, hdg if alpha else None, alpha)
                sdx, sdg = G.rmsnorm_reverse_scales(xh, gh, dyh, 1e-6, hdx if alpha else None, hdg if alpha else None, alpha)
                G.compare(dx.t, rdx, dtype, f"rmsnorm rev wavefront groups dx ({m},{n}) alpha {alpha}", scale=sdx)
                G.compare(dg.t, rdg, dtype, f"rmsnorm rev wavefront groups dg ({m},{n}) alpha {alpha}", rowwise=False, scale=sdg)
                for b in (x, g, dy, dx, dg, scratch):
                    b.check("rmsnorm rev wavefront groups")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_rmsnorm_reverse_three_rows_in_flight_ends_at_every_step(dtype):
    """Short rows run with three register sets that take turns (two rows on their way while a third is
    reduced): row counts that leave the three-step loop after each of its steps, after one to three
    whole turns, on a power-of-two group (128 packs), a three-wavefront group (160) and, for r16, a
    512-thread group (448 packs). Whole problem against the oracle, both blends."""
    r = rng(71)
    per_pack = 16 // torch.empty((), dtype=dtype).element_size()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    for packs, rows_a_group in ((128, 8), (160, 5), (448, 2)):
        n = packs * per_pack
        step = cus * rows_a_group  # rows that one step of every workgroup covers
        for m in (3 * step + 7, 4 * step + 1, 5 * step, 6 * step + step // 2, 9 * step - 1):
            alpha = 0.0 if m % 2 else -0.5
            G.say(f"rmsnorm rev three sets dtype={dtype} ({m},{n}) alpha={alpha}")
            x = G.dev(r.normal(0, 1, (m, n)), dtype)
            g = G.dev(r.normal(1, 0.02, n), dtype)
            dy = G.dev(r.normal(0, 1, (m, n)), dtype)
            dx = G.dev(r.normal(0, 1, (m, n)), dtype)
            dg = G.dev(r.normal(0, 1, n), dtype)
            hdx, hdg = G.host(dx.t).copy(), G.host(dg.t).copy()
            scratch, _ = G.rmsnorm_scratch(dtype, m, n)
            G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, scratch.t, 1e-6, alpha)
            xh, gh, dyh = G.host(x.t), G.host(g.t), G.host(dy.t)
            rdx, rdg = O.rmsnorm_ij_j_reverse(xh, gh, dyh, 1e-6, hdx if alpha else None, hdg if alpha else None, alpha)
            sdx, sdg = G.rmsnorm_reverse_scales(xh, gh, dyh, 1e-6, hdx if alpha else None, hdg if alpha else None, alpha)
            G.compare(dx.t, rdx, dtype, f"rmsnorm rev three sets dx ({m},{n}) alpha {alpha}", scale=sdx)
            G.compare(dg.t, rdg, dtype, f"rmsnorm rev three sets dg ({m},{n}) alpha {alpha}", rowwise=False, scale=sdg)
            for b in (x, g, dy, dx, dg, scratch):
                b.check("rmsnorm rev three sets")


def test_rmsnorm_reverse_long_rows_in_place():
    # dx written over dy: the shared-row path must not be taken
    r = rng(63)
    f32 = torch.float32
    m, n = 3, 151936
    x = G.dev(r.normal(0, 1, (m, n)), f32)
    g = G.dev(r.normal(1, 0.02, n), f32)
    dy = G.dev(r.normal(0, 1, (m, n)), f32)
    dg = G.Guarded((n,), f32)
    rdx, rdg = O.rmsnorm_ij_j_reverse(G.host(x.t), G.host(g.t), G.host(dy.t), 1e-6)
    sdx, sdg = G.rmsnorm_reverse_scales(G.host(x.t), G.host(g.t), G.host(dy.t), 1e-6)
    scratch, _ = G.rmsnorm_scratch(f32, m, n)
    G.say("rmsnorm rev long rows, dx over dy")
    G.rmsnorm_reverse(x.t, g.t, dy.t, dy.t, dg.t, scratch.t, 1e-6, 0.0)
    G.compare(dy.t, rdx, f32, "rmsnorm rev in place dx", scale=sdx)
    G.compare(dg.t, rdg, f32, "rmsnorm rev in place dg", rowwise=False, scale=sdg)
    for gd in (dy, dg, scratch):
        gd.check("rmsnorm rev in place")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_rmsnorm_reverse_unaligned(dtype):
    r = rng(61)
    eps = 1e-6
    for (m, n) in [(5, 100), (3, 1027), (4, 4096), (700, 100), (300, 7), (130, 1003), (9, 9001)]:
        for shifts in [(1, 0, 1, 1), (0, 1, 0, 0), (0, 0, 0, 0)]:
            G.say(f"rmsnorm rev unaligned dtype={dtype} shape=({m},{n}) shifts={shifts}")
            x = G.dev(r.normal(0, 1, (m, n)), dtype, shifts[0])
            g = G.dev(r.normal(1, 0.02, n), dtype, shifts[1])
            dy = G.dev(r.normal(0, 1, (m, n)), dtype, shifts[2])
            dx = G.Guarded((m, n), dtype, shifts[3])
            dg = G.Guarded((n,), dtype)
            scratch, _ = G.rmsnorm_scratch(dtype, m, n)
            G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, scratch.t, eps, 0.0)
            rdx, rdg = O.rmsnorm_ij_j_reverse(G.host(x.t), G.host(g.t), G.host(dy.t), eps)
            sdx, sdg = G.rmsnorm_reverse_scales(G.host(x.t), G.host(g.t), G.host(dy.t), eps)
            G.compare(dx.t, rdx, dtype, f"rmsnorm rev unaligned dx ({m},{n})", scale=sdx)
            G.compare(dg.t, rdg, dtype, f"rmsnorm rev unaligned dg ({m},{n})", rowwise=False, scale=sdg)
            for gd in (dx, dg, scratch):
                gd.check("rmsnorm rev unaligned")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_rmsnorm_short_rows_any_length_and_alignment(dtype):
    """Rows of one element up to sixteen packs and a little beyond, forward and reverse: 1 ... 16
    lanes a row, packs from the row's first element, cut packs in pieces; bases shifted apart,
    the alpha blend, in place, and row counts from three to more than the workgroups hold at once."""
    r = rng(63)
    eps = 1e-6
    lengths = list(range(1, 20)) + [24, 31, 32, 33, 40, 47, 48, 63, 64, 65, 96, 100, 127, 128, 129, 136]
    for n in lengths:
        for (m, shifts) in [(3, (0, 0, 0, 0)), (1001, (1, 0, 3, 2)), (70001 if n <= 8 else 9001, (0, 1, 0, 0))]:
            for alpha in (0.0, 0.5):
                G.say(f"rmsnorm short dtype={dtype} shape=({m},{n}) shifts={shifts} alpha={alpha}")
                x = G.dev(r.normal(0, 1, (m, n)), dtype, shifts[0])
                g = G.dev(r.normal(1, 0.02, n), dtype, shifts[1])
                dy = G.dev(r.normal(0, 1, (m, n)), dtype, shifts[2])
                dx = G.dev(r.normal(0, 1, (m, n)), dtype, shifts[3])
                dg = G.dev(r.normal(0, 1, n), dtype)
                y = G.Guarded((m, n), dtype, shifts[3])
                xh, gh, dyh = G.host(x.t), G.host(g.t), G.host(dy.t)
                hdx, hdg = G.host(dx.t).copy(), G.host(dg.t).copy()
                G.rmsnorm(x.t, g.t, y.t, eps)
                G.compare(y.t, O.rmsnorm_ij_j(xh, gh, eps), dtype, f"rmsnorm short ({m},{n})")
                y.check("y")
                scratch, _ = G.rmsnorm_scratch(dtype, m, n)
                G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, scratch.t, eps, alpha)
                rdx, rdg = O.rmsnorm_ij_j_reverse(xh, gh, dyh, eps, hdx if alpha else None, hdg if alpha else None, alpha)
                sdx, sdg = G.rmsnorm_reverse_scales(xh, gh, dyh, eps, hdx if alpha else None, hdg if alpha else None, alpha)
                G.compare(dx.t, rdx, dtype, f"rmsnorm short dx ({m},{n}) alpha {alpha}", scale=sdx)
                G.compare(dg.t, rdg, dtype, f"rmsnorm short dg ({m},{n}) alpha {alpha}", rowwise=False, scale=sdg)
                for gd in (x, g, dy, dx, dg, scratch):
                    gd.check("rmsnorm short")
            G.rmsnorm(x.t, g.t, x.t, eps)
            G.compare(x.t, O.rmsnorm_ij_j(xh, gh, eps), dtype, f"rmsnorm short in place ({m},{n})")
            x.check("in place")


def test_rmsnorm_reverse_is_deterministic():
    r = rng(62)
    m, n = 2048, 4096
    x = G.dev(r.normal(0, 1, (m, n)), torch.float32)
    g = G.dev(r.normal(1, 0.02, n), torch.float32)
    dy = G.dev(r.normal(0, 1, (m, n)), torch.float32)
    scratch, _ = G.rmsnorm_scratch(torch.float32, m, n)
    outs = []
    for rep in range(3):
        dx = G.Guarded((m, n), torch.float32)
        dg = G.Guarded((n,), torch.float32)
        G.say(f"rmsnorm rev determinism rep {rep}")
        G.rmsnorm_reverse(x.t, g.t, dy.t, dx.t, dg.t, scratch.t, 1e-6, 0.0)
        outs.append((dx.t.clone(), dg.t.clone()))
    for dx, dg in outs[1:]:
        assert torch.equal(dx, outs[0][0]) and torch.equal(dg, outs[0][1])


# ------------------------------------------------------------------ streams

def test_launchers_follow_the_stream_of_the_context():
    kernels, utils = G.lib()
    sc = utils.mpInitStream()
    assert sc.blas_handle.ptr and sc.hip_stream.ptr  # the stream and its BLAS handle
    r = rng(70)
    n = 1 << 20
    a, b = G.dev(r.normal(0, 1, n), torch.float32), G.dev(r.normal(0, 1, n), torch.float32)
    c = G.Guarded((n,), torch.float32)
    torch.cuda.synchronize()
    G.say("addition on an mpInitStream stream")
    kernels.addition[1](a.t.data_ptr(), b.t.data_ptr(), c.t.data_ptr(), n, sc)
    utils.mpStreamSynchronize(sc)
    G.compare(c.t, O.addition(G.host(a.t), G.host(b.t)), torch.float32, "addition on own stream", rowwise=False)
    utils.mpDeinitStream(sc)


def test_shared_rows_on_two_streams_at_once_with_a_workspace_each():
    """Launches that may overlap in time get different workspaces: the workspace is the key under
    which the library keeps a launch's exchange words. Two streams, each with its own workspace
    and its own inputs, enqueue the shared-row softmax forward and reverse ten times without
    waiting for each other; every result against the oracle."""
    kernels, utils = G.lib()
    r = rng(71)
    f32 = torch.float32
    m, n = 48, 50257
    fwd_bytes = G.row_size("mpSoftmaxScratchBytes", f32, m, n)
    rev_bytes = G.row_size("mpSoftmaxReverseScratchBytes", f32, m, n)
    assert fwd_bytes > 0 and rev_bytes > 0
    lanes = []
    for _ in range(2):
        lanes.append(dict(sc=utils.mpInitStream(), fs=G.Guarded((fwd_bytes,), torch.uint8), rs=G.Guarded((rev_bytes,), torch.uint8),
                          x=[G.dev(r.normal(0, 3, (m, n)), f32) for _ in range(2)], dy=G.dev(r.normal(0, 1, (m, n)), f32),
                          y=[G.Guarded((m, n), f32) for _ in range(2)], dx=[G.Guarded((m, n), f32) for _ in range(2)]))
    torch.cuda.synchronize()
    G.say(f"shared rows on two streams ({m},{n})")
    for launch in range(10):
        for ln in lanes:
            k = launch % 2
            kernels.softmax_ij_j[1](ln["x"][k].t.data_ptr(), ln["y"][k].t.data_ptr(), ln["fs"].t.data_ptr(), m, n, ln["sc"])
            kernels.softmax_ij_j_reverse[1](ln["y"][k].t.data_ptr(), ln["dy"].t.data_ptr(), ln["dx"][k].t.data_ptr(),
                                            ln["rs"].t.data_ptr(), 0.0, m, n, ln["sc"])
    for ln in lanes:
        utils.mpStreamSynchronize(ln["sc"])
    for i, ln in enumerate(lanes):
        dyh = G.host(ln["dy"].t)
        for k in range(2):
            yh = G.host(ln["y"][k].t)
            G.compare(ln["y"][k].t, O.softmax_ij_j(G.host(ln["x"][k].t)), f32, f"stream {i} y{k}", atol=1e-6)
            G.compare(ln["dx"][k].t, O.softmax_ij_j_reverse(yh, dyh), f32, f"stream {i} dx{k}", scale=G.softmax_reverse_scale(yh, dyh))
            ln["y"][k].check("y")
            ln["dx"][k].check("dx")
        ln["fs"].check("forward workspace")
        ln["rs"].check("reverse workspace")
        utils.mpDeinitStream(ln["sc"])


def test_device_utils_roundtrip():
    kernels, utils = G.lib()
    utils.mpInitDevice(0)
    assert utils.mpDeviceTotalMemory(0) > (100 << 30)
    sc = utils.mpInitStream()
    src = np.arange(100003, dtype=np.float32)
    dst = np.zeros_like(src)
    G.say("mpMemAlloc / HtoD / DtoH / Free")
    d = utils.mpMemAlloc(src.nbytes, sc)
    assert d
    utils.mpMemcpyHtoD(d, src.ctypes.data, src.nbytes, sc)
    utils.mpMemcpyDtoH(dst.ctypes.data, d, src.nbytes, sc)  # returns with the bytes landed
    assert np.array_equal(src, dst)
    utils.mpMemFree(d, sc)
    utils.mpStreamSynchronize(sc)
    utils.mpDeviceSynchronize()
    utils.mpCheckLastError()
    utils.mpDeinitStream(sc)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=["r32", "r16"])
@pytest.mark.parametrize("n", [96, 2048, 40000], ids=["short", "resident", "long"])
def test_special_values_follow_the_closed_forms(dtype, n):
    """NaN, +inf and all-zero rows: the kernels return what the closed forms (the oracle) return,
    NaN where they are NaN, in every row regime; rows without special values are untouched."""
    r = rng(91)
    m = 6
    x = r.normal(0, 1, (m, n))
    x[1, n // 3] = np.inf          # softmax: exp(inf - inf) -> NaN row; rmsnorm: inf / inf -> NaN
    x[2, n // 2] = np.nan          # NaN spreads over its row only
    x[3, :] = 0.0                  # softmax: uniform 1/n; rmsnorm: 0 * rsqrt(eps) = 0
    x[4, 5] = -np.inf              # softmax: exactly 0 there
    eps = 1e-6
    G.say(f"special values dtype={dtype} n={n}")
    xd = G.dev(x, dtype)
    g = G.dev(r.normal(1, 0.02, n), dtype)
    p, y = G.Guarded((m, n), dtype), G.Guarded((m, n), dtype)
    G.softmax(xd.t, p.t)
    G.rmsnorm(xd.t, g.t, y.t, eps)
    xh = G.host(xd.t)
    with np.errstate(all="ignore"):
        ref_p, ref_y = O.softmax_ij_j(xh), O.rmsnorm_ij_j(xh, G.host(g.t), eps)
    G.compare(p.t, ref_p, dtype, "softmax with special values", **G.softmax_tol(dtype))
    G.compare(y.t, ref_y, dtype, "rmsnorm with special values")
    got_p, got_y = G.host(p.t).astype(np.float64), G.host(y.t).astype(np.float64)
    assert np.array_equal(np.isnan(got_p), np.isnan(ref_p)), "softmax: NaN exactly where the closed form is NaN"
    assert np.array_equal(np.isnan(got_y), np.isnan(ref_y)), "rmsnorm: NaN exactly where the closed form is NaN"
    assert np.isnan(ref_p[1]).all() and np.isnan(ref_p[2]).all() and not np.isnan(ref_p[[0, 3, 4, 5]]).any()
    assert got_p[4, 5] == 0.0 and np.allclose(got_p[3], 1.0 / n, rtol=2e-3)
    assert (got_y[3] == 0.0).all()
    for gd in (xd, g, p, y):
        gd.check("special values")
