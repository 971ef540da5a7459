"""Expressions fused at run time, on the GPU, through the C-ABI of lib/libmp_fusion.so.

Two kinds of evidence. The expressions of chains.json exist twice, compiled into the library at
build time and compiled by hiprtc at run time from the same functor text and the same engine:
their results must agree to the rounding of the storage type, at every operand layout, dtype and
blend (not bit for bit: the two compilations pick fused or separate conversions to r16 differently,
which moves a result at a rounding tie by one unit in the last place). Expressions nobody listed
are checked against torch autograd in fp64 on the same (storage-rounded) inputs. Both bounds scale
with the magnitudes an entry is combined from."""
import numpy as np
import pytest
import torch

import gpu_lib as G
from metaphor_amd import chaingen
from test_chain_fusion import random_expression
from test_chaingen import _torch_eval

pytestmark = pytest.mark.gpu

DTYPES = [torch.float16, torch.float32, torch.float64]
IDS = ["r16", "r32", "r64"]
SIZES = [1, 7, 1000, 4099, (1 << 20) + 5]
LAM, ALP = 1.0507010, 1.6732632


def _static(name, dtype, *args):
    G._call(name, dtype, *args)


ULP = {torch.float16: 2.0 ** -10, torch.float32: 2.0 ** -23, torch.float64: 2.0 ** -52}


def _same_to_rounding(a, b, scale, dtype, what):
    """|a - b| <= 2 units in the last place of the terms the entry is combined from."""
    err = (a.double() - b.double()).abs().cpu().numpy()
    bound = 2.0 * ULP[dtype] * np.maximum(scale, np.abs(b.double().cpu().numpy()))
    bad = err > bound
    exact = float((err == 0).mean()) if err.size else 1.0
    assert not bad.any(), f"{what}: {int(bad.sum())} entries apart by more than rounding (largest {err.max():.3e})"
    return exact


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("chain", chaingen.load_chains(), ids=lambda c: c["name"])
def test_listed_chains_agree_with_their_build_time_kernels(chain, dtype):
    expr, name = chain["expr"], chain["name"]
    root, k = chaingen.parse(expr)
    r = np.random.default_rng(3)
    fewest = 1.0
    for n in SIZES:
        for shifts in ([0] * (2 * k + 2), [1] * (2 * k + 2), [int(v) for v in r.integers(0, 3, 2 * k + 2)]):
            for alpha in (0.0, -0.5):
                G.say(f"chain {name} dtype={dtype} n={n} shifts={shifts} alpha={alpha}")
                xs = [G.dev(r.uniform(-2, 2, n), dtype, shifts[i]) for i in range(k)]
                out_a, out_b = G.Guarded((n,), dtype, shifts[k]), G.Guarded((n,), dtype, shifts[k])
                assert G.chain_forward(expr, [x.t for x in xs], out_a.t) == 0, G.chain_error()
                _static(name, dtype, *[x.t.data_ptr() for x in xs], out_b.t.data_ptr(), n)
                up = G.dev(r.normal(0, 1, n), dtype, shifts[k + 1])
                old = [r.normal(0, 1, n) for _ in range(k)]
                ga = [G.dev(old[i], dtype, shifts[k + 2 + i]) for i in range(k)]
                gb = [G.dev(old[i], dtype, shifts[k + 2 + i]) for i in range(k)]
                hold = [G.host(g.t).astype(np.float64) for g in ga]
                assert G.chain_reverse(expr, [x.t for x in xs], up.t, [g.t for g in ga], alpha) == 0, G.chain_error()
                _static(name + "_reverse", dtype, *[x.t.data_ptr() for x in xs], up.t.data_ptr(),
                        *[g.t.data_ptr() for g in gb], float(alpha), n)
                vmag, gmag = _magnitudes(root, [G.host(x.t) for x in xs], G.host(up.t))
                fewest = min(fewest, _same_to_rounding(out_a.t, out_b.t, vmag, dtype, f"{name} value"))
                for i in range(k):
                    fewest = min(fewest, _same_to_rounding(ga[i].t, gb[i].t, gmag[i] + abs(alpha) * np.abs(hold[i]), dtype,
                                                           f"{name} gradient of leaf {i}"))
                for b in xs + [out_a, out_b, up] + ga + gb:
                    b.check(name)
    print(f"[chain-agreement] {name} {dtype}: at least {fewest:.5f} of the entries of every result are bit-identical")


def _magnitudes(root, leaves, up):
    """Upper bounds, entry by entry, of the terms the value and each leaf gradient are combined
    from: the expression on |leaves| with every op replaced by a bound of its magnitude and slope."""
    bound_op = {"add": torch.add, "sub": torch.add, "mul": torch.mul, "neg": lambda a: a, "relu": lambda a: a,
                "selu": lambda a: LAM * ALP * a}

    def ev(n):
        if n.op == "leaf":
            return ts[n.leaf]
        if n.op == "scale":
            return ev(n.args[0]) * abs(n.constant)
        if n.op == "shift":
            return ev(n.args[0]) + abs(n.constant)
        return bound_op[n.op](*[ev(a) for a in n.args])

    ts = [torch.from_numpy(np.abs(x)).double().requires_grad_(True) for x in leaves]
    v = ev(root)
    v.backward(torch.from_numpy(np.abs(up)).double())
    return v.detach().numpy(), [t.grad.numpy() if t.grad is not None else np.zeros_like(up) for t in ts]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_unlisted_expressions_match_autograd(dtype):
    r = np.random.default_rng(17)
    for case in range(12):
        expr = random_expression(r, int(r.integers(1, 9)), int(r.integers(2, 5)))
        root, k = chaingen.parse(expr)
        n = int(r.choice([5, 777, 70001]))
        shift = int(r.integers(0, 2))
        alpha = float(r.choice([0.0, 1.0, -0.5]))
        G.say(f"unlisted chain {expr} dtype={dtype} n={n} shift={shift} alpha={alpha}")
        xs = [G.dev(r.uniform(-1.5, 1.5, n), dtype, shift) for _ in range(k)]
        up = G.dev(r.normal(0, 1, n), dtype, shift)
        old = [G.dev(r.normal(0, 1, n), dtype, shift) for _ in range(k)]
        hx, hup, hold = [G.host(x.t) for x in xs], G.host(up.t), [G.host(o.t).copy() for o in old]
        out = G.Guarded((n,), dtype, shift)
        assert G.chain_forward(expr, [x.t for x in xs], out.t) == 0, G.chain_error()
        assert G.chain_reverse(expr, [x.t for x in xs], up.t, [o.t for o in old], alpha) == 0, G.chain_error()

        ts = [torch.from_numpy(x.astype(np.float64)).requires_grad_(True) for x in hx]
        ref = _torch_eval(root, ts)
        ref.backward(torch.from_numpy(hup.astype(np.float64)))
        vmag, gmag = _magnitudes(root, hx, hup)
        G.compare(out.t, ref.detach().numpy(), dtype, f"{expr} value", rowwise=False, scale=vmag)
        for i in range(k):
            g = ts[i].grad.numpy() if ts[i].grad is not None else np.zeros(n)
            want = g + alpha * hold[i].astype(np.float64)
            G.compare(old[i].t, want, dtype, f"{expr} gradient of leaf {i}", rowwise=False,
                      scale=gmag[i] + abs(alpha) * np.abs(hold[i].astype(np.float64)))
        for b in xs + [up, out] + old:
            b.check(expr)


def test_output_may_alias_a_leaf_and_empty_and_null_calls_enqueue_nothing():
    r = np.random.default_rng(5)
    f32 = torch.float32
    expr = "sub(mul(0,1),relu(0))"
    a, b = G.dev(r.uniform(-2, 2, 5000), f32), G.dev(r.uniform(-2, 2, 5000), f32)
    ha, hb = G.host(a.t).astype(np.float64), G.host(b.t).astype(np.float64)
    G.say("chain in place")
    assert G.chain_forward(expr, [a.t, b.t], a.t) == 0, G.chain_error()
    G.compare(a.t, ha * hb - np.where(ha >= 0, ha, 0.0), f32, "in place", rowwise=False, scale=np.abs(ha * hb) + np.abs(ha))
    a.check("in place")
    before = a.t.clone()
    empty = a.t[:0]
    assert G.chain_forward(expr, [empty, empty], empty) == 0
    f = G.ffi.load_fusion()
    import ctypes
    ptrs = (ctypes.c_void_p * 2)(a.t.data_ptr(), None)
    assert f.mpChainForward(expr.encode(), 1, ptrs, a.t.data_ptr(), 10, G.ctx()) != 0
    assert "NULL" in G.chain_error()
    assert G.chain_forward("add(0,frob(1))", [a.t, b.t], a.t) != 0
    assert "unknown op" in G.chain_error()
    torch.cuda.synchronize()
    assert torch.equal(a.t, before)


def test_one_kernel_serves_every_value_of_a_constant():
    """relu(c1 * (a * b) + c2) with four pairs of constants: one compilation, every result against
    fp64 numpy on the storage-rounded inputs (a constant reaches the kernel as an argument)."""
    r = np.random.default_rng(9)
    f = G.ffi.load_fusion()
    for dtype in DTYPES:
        n = 30011
        a, b = G.dev(r.uniform(-2, 2, n), dtype), G.dev(r.uniform(-2, 2, n), dtype)
        up = G.dev(r.normal(0, 1, n), dtype)
        ha, hb, hup = (G.host(t.t).astype(np.float64) for t in (a, b, up))
        sizes = set()
        for c1, c2 in [(0.125, 0.5), (-0.75, 0.25), (3.0, -1e-3), (1e-2, 7.0)]:
            expr = f"relu(shift(scale(mul(0,1),{c1!r}),{c2!r}))"
            G.say(f"chain constants dtype={dtype} c1={c1} c2={c2}")
            out = G.Guarded((n,), dtype)
            ga, gb = G.Guarded((n,), dtype), G.Guarded((n,), dtype)
            assert G.chain_forward(expr, [a.t, b.t], out.t) == 0, G.chain_error()
            assert G.chain_reverse(expr, [a.t, b.t], up.t, [ga.t, gb.t], 0.0) == 0, G.chain_error()
            sizes.add(int(f.mpChainCacheSize()))
            pre = c1 * (ha * hb) + c2
            on = (pre >= 0) * hup
            mag = abs(c1) * np.abs(ha * hb) + abs(c2)
            G.compare(out.t, np.where(pre >= 0, pre, 0.0), dtype, f"{expr} value", rowwise=False, scale=mag)
            G.compare(ga.t, on * c1 * hb, dtype, f"{expr} da", rowwise=False, scale=np.abs(hup * c1 * hb))
            G.compare(gb.t, on * c1 * ha, dtype, f"{expr} db", rowwise=False, scale=np.abs(hup * c1 * ha))
            for g in (out, ga, gb):
                g.check(expr)
        assert len(sizes) == 1, "another value of a constant must not be another compilation"


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_several_results_in_one_kernel_match_autograd(dtype):
    """u = a + b; e1 = selu(u * c); e2 = relu(u - d) (and two more texts) as ONE forward kernel with
    as many output streams and ONE reverse kernel that takes both upstream gradients; against torch
    autograd in fp64 on the storage-rounded inputs, overwrite and blend, aligned and shifted."""
    r = np.random.default_rng(23)
    texts = ["selu(mul(add(0,1),2));relu(sub(add(0,1),3))", "mul(0,0);add(0,1);scale(1,0.5)",
             "neg(0);relu(1);selu(mul(0,1));shift(sub(2,0),-0.25)"]
    for text in texts:
        exprs = text.split(";")
        k, R = G.ffi.load_fusion().mpChainLeaves(text.encode()), len(exprs)
        assert G.ffi.load_fusion().mpChainRoots(text.encode()) == R
        for n, shift, alpha in [(5, 0, 0.0), (70001, 0, 0.0), (70001, 1, -0.5), (1 << 20, 0, 1.0)]:
            G.say(f"several results {text} dtype={dtype} n={n} shift={shift} alpha={alpha}")
            xs = [G.dev(r.uniform(-1.5, 1.5, n), dtype, shift) for _ in range(k)]
            ups = [G.dev(r.normal(0, 1, n), dtype, shift) for _ in range(R)]
            old = [G.dev(r.normal(0, 1, n), dtype, shift) for _ in range(k)]
            outs = [G.Guarded((n,), dtype, shift) for _ in range(R)]
            hx, hup, hold = [G.host(x.t) for x in xs], [G.host(u.t) for u in ups], [G.host(o.t).copy() for o in old]
            assert G.chain_forward_many(text, [x.t for x in xs], [o.t for o in outs]) == 0, G.chain_error()
            assert G.chain_reverse_many(text, [x.t for x in xs], [u.t for u in ups], [o.t for o in old], alpha) == 0, G.chain_error()
            ts = [torch.from_numpy(x.astype(np.float64)).requires_grad_(True) for x in hx]
            gmag = [np.zeros(n) for _ in range(k)]
            refs = []
            for e, up in zip(exprs, hup):  # each result with its own leaf numbering for the build-time parser
                names = []
                def local(m):
                    g = int(m.group(1))
                    if g not in names:
                        names.append(g)
                    return f"x{names.index(g)}"
                import re
                root, _ = chaingen.parse(re.sub(r"(?<=[(,])(\d+)(?=[,)])(?!\.)", lambda m: local(m), _leaves_only(e)))
                val = _torch_eval(root, [ts[g] for g in names])
                refs.append(val)
                vmag, gm = _magnitudes(root, [hx[g] for g in names], up)
                for j, g in enumerate(names):
                    gmag[g] = gmag[g] + gm[j]
                refs[-1] = (val, vmag)
            total = sum((v * torch.from_numpy(u.astype(np.float64))).sum() for (v, _), u in zip(refs, hup))
            total.backward()
            for o, (v, vmag) in zip(outs, refs):
                G.compare(o.t, v.detach().numpy(), dtype, f"{text} value", rowwise=False, scale=vmag)
            for i in range(k):
                g = ts[i].grad.numpy() if ts[i].grad is not None else np.zeros(n)
                want = g + alpha * hold[i].astype(np.float64)
                G.compare(old[i].t, want, dtype, f"{text} gradient of leaf {i}", rowwise=False,
                          scale=gmag[i] + abs(alpha) * np.abs(hold[i].astype(np.float64)))
            for b in xs + ups + outs + old:
                b.check(text)


def _leaves_only(e):
    """The text of one result with its constants protected from the leaf renumbering: a constant is the
    second argument of scale / shift."""
    import re
    return re.sub(r"((?:scale|shift)\((?:[^()]|\([^()]*\))*),(-?[\d.]+(?:e-?\d+)?)\)", lambda m: f"{m.group(1)},{float(m.group(2))!r}e0)", e)


def test_forward_variants_that_keep_or_stream_their_inputs_give_the_same_bits():
    """A chain's forward loads inputs that together fit the memory-side cache with ordinary loads (its
    reverse then finds them there) and larger ones, or operands off their 16-byte alignment, with
    streaming loads: the same values either way, build-time and run-time kernels alike. 2^20 elements
    (kept when aligned, streaming one element further) and 17 * 2^20 (four inputs of 68 MiB: beyond
    the cache, streaming)."""
    f32 = torch.float32
    expr = "selu(mul(add(0,1),add(2,3)))"
    r = np.random.default_rng(11)
    for n in (1 << 20, 17 << 20):
        vals = [torch.from_numpy(r.uniform(-2, 2, n).astype(np.float32)).cuda() for _ in range(4)]
        got = []
        for shift in (0, 1):
            xs = [G.Guarded((n,), f32, shift) for _ in range(4)]
            for x, v in zip(xs, vals):
                x.t.copy_(v)
            run_time, build_time = G.Guarded((n,), f32, shift), G.Guarded((n,), f32, shift)
            G.say(f"chain forward variants n={n} shift={shift}")
            assert G.chain_forward(expr, [x.t for x in xs], run_time.t) == 0, G.chain_error()
            _static("fused_selu_hadamard_add_add", f32, *[x.t.data_ptr() for x in xs], build_time.t.data_ptr(), n)
            torch.cuda.synchronize()
            for b in xs + [run_time, build_time]:
                b.check("chain forward variants")
            got.append((run_time.t.clone(), build_time.t.clone()))
            del xs, run_time, build_time
        assert torch.equal(got[0][0], got[1][0]), f"n={n}: the run-time kernel's forward variants differ"
        assert torch.equal(got[0][1], got[1][1]), f"n={n}: the build-time kernel's forward variants differ"
        del got, vals
        torch.cuda.empty_cache()


def test_rate_of_a_run_time_kernel_beside_the_build_time_one():
    """2^26 r32 elements: the run-time kernel of the benchmark chain beside the build-time one (same
    engine, same functor), events around 10 launches each. Printed, not asserted: wall-clock checks
    belong to bench.py (its `chain` workload records the ratio and fails --strict on more than 10 %)."""
    n = 1 << 26
    xs = [torch.empty(n, device="cuda").uniform_(-2, 2) for _ in range(4)]
    out = torch.empty(n, device="cuda")
    expr = "selu(mul(add(0,1),add(2,3)))"

    def timed(fn):
        for _ in range(3):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(10):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / 10

    G.say("chain rate")
    t_run = timed(lambda: G.chain_forward(expr, xs, out))
    t_build = timed(lambda: G.fused(*xs, out))
    print(f"[chain-rate] run-time {t_run * 1e3:.1f} us, build-time {t_build * 1e3:.1f} us, "
          f"ratio {t_run / t_build:.3f}, {20 * n / t_run / 1e6:.0f} GB/s")
