"""The chain generator on the CPU: parsing, signatures, and the generated forward / reverse
arithmetic itself, which is executed line by line in fp64 and compared with torch autograd."""
import re

import numpy as np
import pytest
import torch

import oracle_lib as O
from metaphor_amd import chaingen

torch.set_default_dtype(torch.float64)

def _selu(x):
    """SELU with this workload's truncated constants, differentiable by torch."""
    lam, alp = 1.0507010, 1.6732632
    return torch.where(x > 0, lam * x, lam * alp * torch.expm1(torch.clamp(x, max=0.0)))


def _relu(x):
    """relu with the reference's convention at the kink: slope 1 at exactly 0 (a >= 0 passes the
    gradient, src/cuda/nvcc_src/relu_reverse.cu:12-14); torch.relu takes slope 0 there, and
    half-precision operands hit exact zeros often."""
    return torch.where(x >= 0, x, torch.zeros_like(x))


TORCH_OP = {"add": torch.add, "sub": torch.sub, "mul": torch.mul, "neg": torch.neg,
            "relu": _relu, "selu": _selu}


def _torch_eval(node, leaves):
    if node.op == "leaf":
        return leaves[node.leaf]
    args = [_torch_eval(a, leaves) for a in node.args]
    if node.op == "scale":
        return args[0] * node.constant
    if node.op == "shift":
        return args[0] + node.constant
    return TORCH_OP[node.op](*args)


class _MP:
    """The device helpers the generated lines call, in fp64 (the pinned oracle pieces)."""
    selu_value = staticmethod(lambda x: O.selu(np.asarray(x, dtype=np.float64)))
    selu_slope = staticmethod(lambda x: O.selu_reverse(np.asarray(x, dtype=np.float64), np.ones_like(x)))
    relu_value = staticmethod(lambda x: O.relu(np.asarray(x, dtype=np.float64)))
    relu_slope = staticmethod(lambda x: O.stepwise(np.asarray(x, dtype=np.float64)))


def _run_lines(lines, inputs):
    env = {"inp": inputs, "mp": _MP}
    for line in lines:
        stmt = line.strip().rstrip(";").replace("const P ", "").replace("mp::", "mp.").replace("(P)(", "(")
        stmt = re.sub(r"\bin\[", "inp[", stmt)
        exec(stmt, {}, env)
    return env


@pytest.mark.parametrize("expr", [c["expr"] for c in chaingen.load_chains()] + [
    "mul(add(x0,x0),x1)", "relu(sub(mul(x0,x1),neg(x0)))", "selu(selu(add(x0,x1)))",
    "selu(scale(mul(shift(x0,-1.5),x1),0.1))", "shift(scale(x0,3),2.5e-1)"])
def test_generated_arithmetic_matches_autograd(expr):
    root, k = chaingen.parse(expr)
    rng = np.random.default_rng(5)
    xs = [rng.uniform(-2, 2, 400) for _ in range(k)]
    up = rng.normal(0, 1, 400)
    ts = [torch.from_numpy(x.copy()).requires_grad_(True) for x in xs]
    out = _torch_eval(root, ts)
    out.backward(torch.from_numpy(up.copy()))

    lines, value, _ = chaingen._forward_lines(root)
    env = _run_lines(lines, xs)
    got = eval(re.sub(r"\bin\[", "inp[", value), {}, env)
    np.testing.assert_allclose(got, out.detach().numpy(), rtol=1e-12, atol=1e-14)

    lines, grads = chaingen._reverse_lines(root, k)
    env = _run_lines(lines, xs + [up])
    for i in range(k):
        g = eval(re.sub(r"\bin\[", "inp[", grads[i]), {}, env)
        ref = ts[i].grad.numpy()
        kink = np.zeros_like(ref, dtype=bool)  # torch takes slope 0 at relu(0); none drawn here
        np.testing.assert_allclose(g[~kink], ref[~kink], rtol=1e-12, atol=1e-14)


def test_signatures_number_leaves_in_order_of_first_appearance():
    root, k = chaingen.parse("selu(mul(add(x0,x1),add(x2,x3)))")
    assert (root.signature(), k) == ("selu(mul(add(0,1),add(2,3)))", 4)
    root, k = chaingen.parse("mul(add(x0,x0),x1)")
    assert (root.signature(), k) == ("mul(add(0,0),1)", 2)
    root, k = chaingen.parse("selu(scale(mul(shift(x0, -1.5), x1), 0.1))")
    assert (root.signature(), k) == ("selu(scale(mul(shift(0,-1.5),1),0.10000000000000001))", 2)


@pytest.mark.parametrize("bad", ["x0", "add(x0)", "add(x0,x1,x2)", "foo(x0)", "add(x1,x0)", "add(x0,x2)",
                                 "add(x0,x1))", "add(x0 x1)", "scale(x0)", "scale(x0,x1)", "shift(x0,1,2)", "add(x0,0.5)"])
def test_bad_expressions_are_rejected(bad):
    with pytest.raises(ValueError):
        chaingen.parse(bad)


def test_committed_sources_and_host_table_are_current():
    assert chaingen.generate() == []


def test_generated_sources_obey_the_generator_constraints():
    for c in chaingen.load_chains():
        for text in (chaingen.forward_source(c["name"], c["expr"]), chaingen.reverse_source(c["name"], c["expr"])):
            assert len(re.findall(r"void (launch_\w+)", text)) == 1
            assert "Scalar" in text
            proto = re.search(r'extern "C" void \w+\s?\(([^)]+)\)', text)
            assert proto and ")" not in proto.group(1)
