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


def _literal_constants(expr):
    """The constants of an expression in the order their ops close in the text, which is the order
    the run-time generator numbers them in (c[0], c[1], ...)."""
    return [m.group(1) for m in re.finditer(r",\s*([-+]?(?:\d+\.?\d*|\.\d+)(?:[eE][-+]?\d+)?)\s*\)", expr)
            if True]


def _with_literals(lines, expr):
    """Lines of the run-time generator with each (P)c[i] replaced by the literal the build-time
    generator writes in its place."""
    values = [chaingen.constant_text(float(v)) for v in _literal_constants(expr)]
    return [re.sub(r"\(P\)c\[(\d+)\]", lambda m: f"(P)({values[int(m.group(1))]})", l) for l in lines]


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
    # the run-time kernels take their constants as arguments (c[i]); with the literals put back the
    # arithmetic is the build-time generator's, line for line
    assert _with_literals(got["ChainForward"], expr) == want_f["CFn_Scalar"]
    assert _with_literals(got["ChainReverseOverwrite"], expr) == want_r["CReverseOverwriteFn_Scalar"]
    assert _with_literals(got["ChainReverseBlend"], expr) == want_r["CReverseBlendFn_Scalar"]
    assert "double c[8];" in src.decode()


def test_random_expressions_differentiate_like_autograd():
    lib = ffi.load_fusion()
    r = np.random.default_rng(7)
    for case in range(40):
        expr = random_expression(r, int(r.integers(1, 9)), int(r.integers(1, 5)))
        root, k = chaingen.parse(expr)
        assert lib.mpChainLeaves(expr.encode()) == k
        src = lib.mpChainSource(expr.encode(), 2)
        assert src, (expr, lib.mpChainError())
        bodies = {name: _with_literals(lines, expr) for name, lines in _functor_bodies(src.decode()).items()}
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
    src = lib.mpChainSource(expr, dtype).decode()
    assert f"typedef {kinds[dtype]} ChainT;" in src
    # three operand layouts a direction, and the forward once more with loads that keep its inputs in cache
    assert src.count("MP_CHAIN_KERNEL(chain_forward_") == 4 and "MP_CHAIN_KERNEL(chain_forward_3, mp::EW_KEPT" in src
    assert src.count("MP_CHAIN_KERNEL(chain_reverse_overwrite_") == 3 and src.count("MP_CHAIN_KERNEL(chain_reverse_blend_") == 3


@pytest.mark.parametrize("bad,why", [
    ("0", "bare leaf"), ("add(0)", "expected ','"), ("add(0,1,2)", "expected ')'"), ("foo(0)", "unknown op"),
    ("add(1,0)", "order of first appearance"), ("add(0,2)", "order of first appearance"),
    ("add(0,1))", "trailing text"), ("add(0 1)", "expected ','"), ("", "unknown op"),
    ("add(add(add(add(0,1),add(2,3)),add(add(4,5),add(6,7))),8)", "more than 8 leaves"),
    ("scale(0)", "expected ','"), ("scale(0,x1)", "finite number"), ("shift(0,abc)", "finite number"), ("scale(0,inf)", "finite number"),
    ("shift(" * 9 + "0" + ",1)" * 9, "more than 8 constants"),
    ("neg(" * 65 + "0" + ")" * 65, "more than 64 nodes"), ("neg(" * 100000 + "0" + ")" * 100000, "more than 64 nodes"),
    ("add(0,1);", "unknown op"), ("add(0,1);0", "bare leaf"), ("add(0,1);add(0,3)", "order of first appearance"),
    (";".join(["neg(0)"] * 5), "more than 4 results")])
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
                                    "mpChainSource", "mpChainCodeObject", "mpChainCacheSize", "mpChainCompilations",
                                    "mpChainError", "mpChainForwardMany", "mpChainReverseMany", "mpChainRoots"])
    for n in names:
        assert getattr(lib, n)


def test_several_threads_compile_at_once():
    """Eight threads ask for four new expressions, two threads an expression: every call succeeds, each
    expression is compiled once, and a thread's error text is its own."""
    import threading
    lib = ffi.load_fusion()
    exprs = [f"relu(shift({op}(0,1),0.25))".encode() for op in ("mul", "add", "sub")] + [b"neg(shift(mul(0,1),0.25))"]
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


def test_constants_are_arguments_not_part_of_the_kernel():
    """Expressions that differ in their constants only are one cache entry and one compilation."""
    lib = ffi.load_fusion()
    assert lib.mpChainCompile(b"selu(scale(add(0,1),0.5))", 1) == 0, lib.mpChainError()
    n, started = lib.mpChainCacheSize(), lib.mpChainCompilations()
    for value in ("0.25", "-3", "1e-3", "7.5e2"):
        assert lib.mpChainCompile(f"selu(scale(add(0,1),{value}))".encode(), 1) == 0
    assert lib.mpChainCacheSize() == n and lib.mpChainCompilations() == started
    a = lib.mpChainSource(b"selu(scale(add(0,1),0.5))", 1)
    b = lib.mpChainSource(b"selu(scale(add(0,1),-3))", 1)
    assert a == b and b"c[0]" in a and b"0.5" not in a.split(b"namespace {")[1].split(b"}  // namespace")[0]


def test_a_failed_compilation_is_not_tried_again():
    """With the library's test hook set every compilation fails; the second call for the same
    expression returns the first one's reason without starting another compilation. Run in a child
    process so that the hook does not reach the other tests."""
    import subprocess
    import sys
    code = (
        "import os, sys\n"
        "os.environ['MP_CHAIN_BREAK_COMPILE'] = '1'\n"
        f"sys.path.insert(0, {ffi.ROOT!r})\n"
        "from metaphor_amd import ffi\n"
        "lib = ffi.load_fusion()\n"
        "e = b'relu(mul(neg(0),add(1,0)))'\n"
        "assert lib.mpChainCompile(e, 1) != 0\n"
        "first = lib.mpChainError().decode()\n"
        "assert 'MP_CHAIN_BREAK_COMPILE' in first, first\n"
        "started = lib.mpChainCompilations()\n"
        "assert started == 1\n"
        "assert lib.mpChainCompile(e, 1) != 0 and lib.mpChainError().decode() == first\n"
        "assert lib.mpChainCodeObject(e, 1, None) is None\n"
        "assert lib.mpChainCompilations() == started\n"
        "assert lib.mpChainCacheSize() == 0\n"
        "assert lib.mpChainSource(e, 1)\n"
        "print('ok')\n")
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and "ok" in res.stdout, res.stderr[-2000:]


def test_expressions_with_several_results_differentiate_like_autograd():
    """Up to four results over shared leaves in one text: the forward functor writes every result, the
    reverse functor adds every result's contribution to each leaf (upstream gradient r is in[k + r]),
    a leaf that only some results use gets only theirs; executed line by line against torch autograd."""
    lib = ffi.load_fusion()
    r = np.random.default_rng(11)
    fixed = ["selu(mul(add(x0,x1),x2));relu(sub(add(x0,x1),x3))", "neg(x0);neg(x1)", "mul(x0,x0);add(x0,x1);scale(x1,0.5)"]
    for case in range(30):
        if case < len(fixed):
            text = fixed[case]
        else:  # random trees, leaves renumbered across the whole text as the parser wants them
            roots = int(r.integers(2, 5))
            parts, seen = [], []
            for _ in range(roots):
                e = random_expression(r, int(r.integers(1, 4)), int(r.integers(1, 4)))
                pick = {}
                def renumber(m):
                    old = int(m.group(1))
                    if old not in pick:  # reuse a leaf of an earlier result half of the time
                        pick[old] = int(r.choice(seen)) if seen and r.random() < 0.5 else None
                    if pick[old] is None:
                        pick[old] = len(seen)
                        seen.append(len(seen))
                    return f"x{pick[old]}"
                parts.append(re.sub(r"x(\d+)", renumber, e))
            if len(seen) > 8:
                continue
            text = ";".join(parts)
        exprs = text.split(";")
        assert lib.mpChainRoots(text.encode()) == len(exprs), (text, lib.mpChainError())
        k = lib.mpChainLeaves(text.encode())
        assert k >= 1, (text, lib.mpChainError())
        src = lib.mpChainSource(text.encode(), 2)
        assert src, (text, lib.mpChainError())
        bodies = {name: _with_literals(lines, text) for name, lines in _functor_bodies(src.decode()).items()}
        R = len(exprs)
        xs = [r.uniform(-2, 2, 100) for _ in range(k)]
        ups = [r.normal(0, 1, 100) for _ in range(R)]
        old = [r.normal(0, 1, 100) for _ in range(k)]
        ts = [torch.from_numpy(x.copy()).requires_grad_(True) for x in xs]
        outs = []
        for e in exprs:  # each result parsed by the build-time parser with its own leaf numbering
            names = []
            def local(m):
                g = int(m.group(1))
                if g not in names:
                    names.append(g)
                return f"x{names.index(g)}"
            e_x = e
            root, _ = chaingen.parse(re.sub(r"x(\d+)", local, e_x))
            outs.append(_torch_eval(root, [ts[g] for g in names]))
        total = sum((o * torch.from_numpy(u)).sum() for o, u in zip(outs, ups))
        total.backward()

        fwd_lines = bodies["ChainForward"]
        env = _run_lines([l for l in fwd_lines if not l.startswith("out[")], xs)
        got = [eval(re.sub(r"\bin\[", "inp[", l.split("=", 1)[1].rstrip(";")), {}, env) for l in fwd_lines if l.startswith("out[")]
        assert len(got) == R
        for o, ref in zip(got, outs):
            np.testing.assert_allclose(o, ref.detach().numpy(), rtol=1e-12, atol=1e-14, err_msg=text)
        alpha = 0.25
        rev = bodies["ChainReverseBlend"]
        env = _run_lines([l for l in rev if not l.startswith("out[") and not l.startswith("const P al")], xs + ups + old)
        env["al"] = alpha
        grads = [l for l in rev if l.startswith("out[")]
        assert len(grads) == k
        for i, line in enumerate(grads):
            g = eval(re.sub(r"\bin\[", "inp[", line.split("=", 1)[1].rstrip(";").replace("(P)0", "0.0")), {}, env)
            ref = (ts[i].grad.numpy() if ts[i].grad is not None else 0.0) + alpha * old[i]
            np.testing.assert_allclose(g, ref, rtol=1e-12, atol=1e-13, err_msg=f"{text} leaf {i}")
    # one compilation for the lot, and the single-result entry points refuse it
    assert lib.mpChainCompile(fixed[0].encode(), 1) == 0, lib.mpChainError()
    ctx = ffi.StreamContext()
    import ctypes
    ptrs = (ctypes.c_void_p * 4)()
    assert lib.mpChainForward(fixed[0].encode(), 1, ptrs, None, 16, ctx) != 0
    assert "mpChainForwardMany" in lib.mpChainError().decode()
