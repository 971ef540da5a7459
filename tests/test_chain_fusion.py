"""Expressions fused at run time (lib/libmp_fusion.so) on the CPU: the C++ generator writes the same
arithmetic, line for line, as the build-time generator whose lines test_chaingen.py executes
against torch autograd; random expressions are executed the same way here; every dtype compiles
with hiprtc (which needs no GPU); bad text is refused with a reason and nothing cached."""
import re

import numpy as np
import pytest
import torch

from metaphor_amd import chaingen, ffi
from test_chaingen import _run_lines, _torch_eval

torch.set_default_dtype(torch.float64)

EXTRA = ["mul(add(x0,x0),x1)", "relu(sub(mul(x0,x1),neg(x0)))", "selu(selu(add(x0,x1)))", "neg(x0)",
         "selu(scale(mul(shift(x0,-1.5),x1),0.1))", "shift(scale(x0,3),2.5e-1)",
         "sub(mul(x0,x1),mul(x2,add(x3,add(x4,add(x5,add(x6,x7))))))"]


def _functor_bodies(source):
    """{functor name: [stripped statement lines]} of a generated source."""
    out = {}
    for name, body in re.findall(r"struct (\w+) \{.*?apply\([^)]*\)[^{]*\{\n(.*?)\n  \}\n\};", source, flags=re.S):
        out[name] = [l.strip() for l in body.splitlines() if l.strip()]
    return out


def random_expression(r, leaves, depth):
    """A random tree over the six ops that uses leaves 0..leaves-1 in order of first appearance."""
    used = []

    def leaf():
        k = int(r.integers(0, min(len(used) + 1, leaves)))
        if k == len(used):
            used.append(k)
        return f"x{k}"

    def node(d):
        if d == 0 or (d < depth and r.random() < 0.25):
            return leaf()
        op = str(r.choice(["add", "sub", "mul", "neg", "relu", "selu", "scale", "shift"]))
        if op in ("neg", "relu", "selu"):
            return f"{op}({node(d - 1)})"
        if op in ("scale", "shift"):
            return f"{op}({node(d - 1)},{float(r.choice([0.5, -1.25, 3.0, 0.1, 1e-3])):.17g})"
        return f"{op}({node(d - 1)},{node(d - 1)})"

    text = node(depth)
    return text if "(" in text else f"neg({text})"


@pytest.mark.parametrize("expr", [c["expr"] for c in chaingen.load_chains()] + EXTRA)
def test_the_runtime_generator_writes_the_build_time_generators_lines(expr):
    lib = ffi.load_fusion()
    src = lib.mpChainSource(expr.encode(), 1)
    assert src, lib.mpChainError()
    got = _functor_bodies(src.decode())
    want_f = _functor_bodies(chaingen.forward_source("c", expr))
    want_r = _functor_bodies(chaingen.reverse_source("c", expr))
    assert got["ChainForward"] == want_f["CFn_Scalar"]
    assert got["ChainReverseOverwrite"] == want_r["CReverseOverwriteFn_Scalar"]
    assert got["ChainReverseBlend"] == want_r["CReverseBlendFn_Scalar"]


def test_random_expressions_differentiate_like_autograd():
    lib = ffi.load_fusion()
    r = np.random.default_rng(7)
    for case in range(40):
        expr = random_expression(r, int(r.integers(1, 9)), int(r.integers(1, 5)))
        root, k = chaingen.parse(expr)
        assert lib.mpChainLeaves(expr.encode()) == k
        src = lib.mpChainSource(expr.encode(), 2)
        assert src, (expr, lib.mpChainError())
        bodies = _functor_bodies(src.decode())
        xs = [r.uniform(-2, 2, 200) for _ in range(k)]
        up = r.normal(0, 1, 200)
        old = [r.normal(0, 1, 200) for _ in range(k)]
        ts = [torch.from_numpy(x.copy()).requires_grad_(True) for x in xs]
        out = _torch_eval(root, ts)
        out.backward(torch.from_numpy(up.copy()))

        env = _run_lines([l for l in bodies["ChainForward"] if not l.startswith("out[")], xs)
        fwd = [l for l in bodies["ChainForward"] if l.startswith("out[")]
        assert len(fwd) == 1
        got = eval(re.sub(r"\bin\[", "inp[", fwd[0].split("=", 1)[1].rstrip(";")), {}, env)
        np.testing.assert_allclose(got, out.detach().numpy(), rtol=1e-12, atol=1e-14, err_msg=expr)

        alpha = -0.5
        env = _run_lines([l for l in bodies["ChainReverseBlend"] if not l.startswith("out[")
                          and not l.startswith("const P al")], xs + [up] + old)
        env["al"] = alpha
        outs = [l for l in bodies["ChainReverseBlend"] if l.startswith("out[")]
        assert len(outs) == k
        for i, line in enumerate(outs):
            g = eval(re.sub(r"\bin\[", "inp[", line.split("=", 1)[1].rstrip(";")), {}, env)
            ref = (ts[i].grad.numpy() if ts[i].grad is not None else 0.0) + alpha * old[i]
            np.testing.assert_allclose(g, ref, rtol=1e-12, atol=1e-13, err_msg=f"{expr} leaf {i}")


@pytest.mark.parametrize("dtype", [0, 1, 2], ids=["r16", "r32", "r64"])
def test_every_dtype_compiles_and_is_cached_once(dtype):
    lib = ffi.load_fusion()
    expr = b"relu(mul(sub(0,1),selu(add(2,0))))"
    assert lib.mpChainCompile(expr, dtype) == 0, lib.mpChainError()
    n = lib.mpChainCacheSize()
    # the same expression spelled with x-names and blanks is the same cache entry
    assert lib.mpChainCompile(b"relu( mul(sub(x0, x1), selu(add(x2,x0))) )", dtype) == 0
    assert lib.mpChainCacheSize() == n
    kinds = {0: "_Float16", 1: "float", 2: "double"}
    assert f"typedef {kinds[dtype]} ChainT;" in lib.mpChainSource(expr, dtype).decode()


@pytest.mark.parametrize("bad,why", [
    ("0", "bare leaf"), ("add(0)", "expected ','"), ("add(0,1,2)", "expected ')'"), ("foo(0)", "unknown op"),
    ("add(1,0)", "order of first appearance"), ("add(0,2)", "order of first appearance"),
    ("add(0,1))", "trailing text"), ("add(0 1)", "expected ','"), ("", "unknown op"),
    ("add(add(add(add(0,1),add(2,3)),add(add(4,5),add(6,7))),8)", "more than 8 leaves"),
    ("scale(0)", "expected ','"), ("scale(0,x1)", "finite number"), ("shift(0,abc)", "finite number"), ("scale(0,inf)", "finite number")])
def test_bad_expressions_are_refused_with_a_reason(bad, why):
    lib = ffi.load_fusion()
    n = lib.mpChainCacheSize()
    assert lib.mpChainCompile(bad.encode(), 1) != 0
    assert why in lib.mpChainError().decode()
    assert lib.mpChainLeaves(bad.encode()) == -1
    assert lib.mpChainSource(bad.encode(), 1) is None
    assert lib.mpChainCacheSize() == n


def test_an_unknown_dtype_is_refused():
    lib = ffi.load_fusion()
    assert lib.mpChainCompile(b"add(0,1)", 3) != 0
    assert "dtype" in lib.mpChainError().decode()


def test_the_fusion_library_exports_what_its_header_declares():
    lib = ffi.load_fusion()
    names = [n for _, n, _ in ffi.parse_declarations(ffi.os.path.join(ffi.ROOT, "include", "chain_fusion.h"))]
    assert sorted(names) == sorted(["mpChainForward", "mpChainReverse", "mpChainCompile", "mpChainLeaves",
                                    "mpChainSource", "mpChainCodeObject", "mpChainCacheSize", "mpChainError"])
    for n in names:
        assert getattr(lib, n)


def test_several_threads_compile_at_once():
    """Eight threads ask for four new expressions, two threads an expression: every call succeeds, each
    expression is compiled once, and a thread's error text is its own."""
    import threading
    lib = ffi.load_fusion()
    exprs = [f"relu(shift(mul(0,1),{k}.25))".encode() for k in range(4)]
    before = lib.mpChainCacheSize()
    results = [None] * 8

    def work(i):
        if i == 7:  # one thread fails meanwhile; the others must not see its error
            results[i] = (lib.mpChainCompile(b"foo(0)", 1), lib.mpChainError().decode())
        else:
            results[i] = (lib.mpChainCompile(exprs[i % 4], 1), lib.mpChainError().decode())

    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert [r[0] for r in results[:7]] == [0] * 7, results
    assert results[7][0] != 0 and "unknown op" in results[7][1]
    assert all("unknown op" not in r[1] for r in results[:7])
    assert lib.mpChainCacheSize() == before + 4


def test_missing_operand_arrays_are_refused():
    """No array of leaf pointers: refused before anything touches a device."""
    lib = ffi.load_fusion()
    ctx = ffi.StreamContext()
    assert lib.mpChainForward(b"add(0,1)", 1, None, None, 16, ctx) != 0
    assert "operand array" in lib.mpChainError().decode()
    assert lib.mpChainReverse(b"add(0,1)", 1, None, None, None, 0.0, 16, ctx) != 0
    assert "operand array" in lib.mpChainError().decode()
