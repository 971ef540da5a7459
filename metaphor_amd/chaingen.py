"""Fused elementwise chains: from an expression to HIP kernel sources.

``chains.json`` lists elementwise expressions over leaves ``x0, x1, ...`` built from
``add, sub, mul, neg, relu, selu`` and, with a literal constant as second argument, ``scale`` (the
reference's dilate, x * c) and ``shift`` (its translate, x + c). For every entry this module writes two kernel sources into
``csrc/hipcc_src`` — ``<name>.hip`` (forward, one pass) and ``<name>_reverse.hip`` (all leaf
gradients in one pass, obtained by reverse-mode differentiation of the expression tree) — in the
form the rest of the generator expects: written against ``Scalar``, one launcher per file.
It also writes ``host/chains.hpp``, the table the C++ host side matches pending expressions
against. The reference builds such chains from one kernel and one temporary per op
(README.md:89-97, src/ops/addition.zig:37-47); here a chain costs one read of each leaf and one
write of the result, and its reverse one read of each leaf and of the upstream gradient and one
write per leaf gradient.

ABI of a generated chain with k leaves:
    launch_<name>_<T>(x0, ..., x{k-1}, out, N, ctx)
    launch_<name>_reverse_<T>(x0, ..., x{k-1}, out_grads, g0, ..., g{k-1}, alpha, N, ctx)
with g_i = d out / d x_i * out_grads + alpha * g_i (alpha == 0 never reads g_i).
"""
import json
import os
import re

PKG = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(PKG, "csrc", "hipcc_src")
HOST_DIR = os.path.join(PKG, "host")
ZIG_OPS = os.path.join(os.path.dirname(PKG), "zig", "src", "ops")
CHAINS = os.path.join(PKG, "chains.json")

ARITY = {"add": 2, "sub": 2, "mul": 2, "neg": 1, "relu": 1, "selu": 1, "scale": 1, "shift": 1}
WITH_CONSTANT = ("scale", "shift")  # one tensor argument and one literal: scale(x0,0.5)
MAX_LEAVES = 8

_NUMBER = r"[-+]?(?:\d+\.?\d*|\.\d+)(?:[eE][-+]?\d+)?"
_TOKEN = re.compile(r"\s*([A-Za-z_]\w*|\(|\)|,|" + _NUMBER + ")")


def constant_text(value):
    """How a constant is spelled in signatures and in generated code: the same in every generator."""
    return "%.17g" % float(value)


class Node:
    def __init__(self, op, args=(), leaf=None, constant=None):
        self.op, self.args, self.leaf, self.constant = op, list(args), leaf, constant

    def signature(self):
        """Canonical text the host side builds from a pending tree: leaves are bare indices."""
        if self.op == "leaf":
            return str(self.leaf)
        inner = ",".join(a.signature() for a in self.args)
        if self.op in WITH_CONSTANT:
            inner += "," + constant_text(self.constant)
        return f"{self.op}({inner})"


def parse(expr):
    tokens = _TOKEN.findall(expr)
    if "".join(tokens) != re.sub(r"\s+", "", expr):
        raise ValueError(f"cannot tokenise {expr!r}")
    pos = 0

    def take(expected=None):
        nonlocal pos
        if pos >= len(tokens):
            raise ValueError(f"unexpected end of {expr!r}")
        tok = tokens[pos]
        if expected is not None and tok != expected:
            raise ValueError(f"expected {expected!r}, found {tok!r} in {expr!r}")
        pos += 1
        return tok

    def node():
        tok = take()
        m = re.fullmatch(r"x(\d+)", tok)
        if m:
            return Node("leaf", leaf=int(m.group(1)))
        if tok not in ARITY:
            raise ValueError(f"unknown op {tok!r} in {expr!r}")
        take("(")
        args = [node()]
        while len(args) < ARITY[tok]:
            take(",")
            args.append(node())
        constant = None
        if tok in WITH_CONSTANT:
            take(",")
            literal = take()
            if not re.fullmatch(_NUMBER, literal):
                raise ValueError(f"{tok} wants a number as second argument, found {literal!r} in {expr!r}")
            constant = float(literal)
        take(")")
        return Node(tok, args, constant=constant)

    root = node()
    if pos != len(tokens):
        raise ValueError(f"trailing text in {expr!r}")
    leaves = sorted({n.leaf for n in walk(root) if n.op == "leaf"})
    if leaves != list(range(len(leaves))):
        raise ValueError(f"{expr!r}: leaves must be x0..x{len(leaves) - 1} without gaps")
    order = []
    for n in walk(root):  # first-visit order must be 0, 1, 2, ... as the host numbers leaves
        if n.op == "leaf" and n.leaf not in order:
            order.append(n.leaf)
    if order != leaves:
        raise ValueError(f"{expr!r}: number the leaves in order of first appearance")
    if not 1 <= len(leaves) <= MAX_LEAVES:
        raise ValueError(f"{expr!r}: between 1 and {MAX_LEAVES} leaves")
    if root.op == "leaf":
        raise ValueError(f"{expr!r}: a bare leaf is not a chain")
    return root, len(leaves)


def walk(n):
    """Pre-order, arguments left to right."""
    yield n
    for a in n.args:
        yield from walk(a)


def _forward_lines(root):
    """Post-order temporaries; returns (lines, name of the root value, {id(node): name})."""
    lines, names, counter = [], {}, [0]

    def emit(n):
        if n.op == "leaf":
            names[id(n)] = f"in[{n.leaf}]"
            return names[id(n)]
        a = [emit(c) for c in n.args]
        name = f"t{counter[0]}"
        counter[0] += 1
        rhs = {
            "add": lambda: f"{a[0]} + {a[1]}",
            "sub": lambda: f"{a[0]} - {a[1]}",
            "mul": lambda: f"{a[0]} * {a[1]}",
            "neg": lambda: f"-{a[0]}",
            "relu": lambda: f"mp::relu_value({a[0]})",
            "selu": lambda: f"mp::selu_value({a[0]})",
            "scale": lambda: f"{a[0]} * (P)({constant_text(n.constant)})",
            "shift": lambda: f"{a[0]} + (P)({constant_text(n.constant)})",
        }[n.op]()
        lines.append(f"    const P {name} = {rhs};")
        names[id(n)] = name
        return name

    return lines, emit(root), names


def _reverse_lines(root, k):
    """Reverse-mode sweep: adjoint of the root is in[k]; returns the lines and the leaf adjoints."""
    fwd, _, names = _forward_lines(root)
    lines = list(fwd[:-1])  # no adjoint rule needs the root's own value
    leaf_terms = {i: [] for i in range(k)}
    counter = [0]

    def sweep(n, a):
        if n.op == "leaf":
            leaf_terms[n.leaf].append(a)
            return
        v = [names[id(c)] for c in n.args]

        def fresh(expr):
            name = f"a{counter[0]}"
            counter[0] += 1
            lines.append(f"    const P {name} = {expr};")
            return name

        if n.op == "add":
            sweep(n.args[0], a)
            sweep(n.args[1], a)
        elif n.op == "sub":
            sweep(n.args[0], a)
            sweep(n.args[1], fresh(f"-{a}"))
        elif n.op == "mul":
            sweep(n.args[0], fresh(f"{a} * {v[1]}"))
            sweep(n.args[1], fresh(f"{a} * {v[0]}"))
        elif n.op == "neg":
            sweep(n.args[0], fresh(f"-{a}"))
        elif n.op == "relu":
            sweep(n.args[0], fresh(f"{a} * mp::relu_slope({v[0]})"))
        elif n.op == "selu":
            sweep(n.args[0], fresh(f"{a} * mp::selu_slope({v[0]})"))
        elif n.op == "scale":
            sweep(n.args[0], fresh(f"{a} * (P)({constant_text(n.constant)})"))
        elif n.op == "shift":
            sweep(n.args[0], a)

    sweep(root, f"in[{k}]")
    grads = [" + ".join(leaf_terms[i]) for i in range(k)]
    return lines, grads


def _camel(name):
    return "".join(p.capitalize() for p in name.split("_"))


def forward_source(name, expr):
    root, k = parse(expr)
    lines, value, _ = _forward_lines(root)
    params = "".join(f"  const void* x{i},\n" for i in range(k))
    ins = ", ".join(f"x{i}" for i in range(k))
    return f"""// GENERATED by metaphor_amd/chaingen.py from chains.json -- do not edit.
#include "../elementwise.h"

struct {_camel(name)}Fn_Scalar {{
  template <class P> __device__ __forceinline__ void apply(const P (&in)[{k}], P (&out)[1]) const {{
{chr(10).join(lines)}
    out[0] = {value};
  }}
}};

// out = {expr} in one pass: {k} reads and 1 write per element, where the reference's
// composition takes one launch and one temporary per op (README.md:89-97,
// src/ops/addition.zig:37-47).
extern "C" void launch_{name}_Scalar(
{params}  void* out,
  len_t N,
  StreamContext stream
) {{
  const mp::EwPtrs<{k}, 1> ptrs{{{{{ins}}}, {{out}}}};
  mp::ew_launch_forward<Scalar, {k}, 1, 1>(ptrs, N, {_camel(name)}Fn_Scalar{{}}, get_stream(stream));
}}
"""


def reverse_source(name, expr):
    root, k = parse(expr)
    lines, grads = _reverse_lines(root, k)
    body = "\n".join(lines)
    over = "\n".join(f"    out[{i}] = {grads[i]};" for i in range(k))
    blend = "\n".join(f"    out[{i}] = {grads[i]} + al * in[{k + 1 + i}];" for i in range(k))
    xs = "".join(f"  const void* x{i},\n" for i in range(k))
    gs = "".join(f"  void* g{i},\n" for i in range(k))
    ins = ", ".join(f"x{i}" for i in range(k))
    outs = ", ".join(f"g{i}" for i in range(k))
    cn = _camel(name)
    return f"""// GENERATED by metaphor_amd/chaingen.py from chains.json -- do not edit.
#include "../elementwise.h"

struct {cn}ReverseOverwriteFn_Scalar {{
  template <class P> __device__ __forceinline__ void apply(const P (&in)[{k + 1}], P (&out)[{k}]) const {{
{body}
{over}
  }}
}};

struct {cn}ReverseBlendFn_Scalar {{
  double alpha;
  template <class P> __device__ __forceinline__ void apply(const P (&in)[{2 * k + 1}], P (&out)[{k}]) const {{
    const P al = (P)alpha;
{body}
{blend}
  }}
}};

// Reverse of out = {expr} in one pass: every leaf gradient
// g_i = d out / d x_i * out_grads + alpha * g_i (the blend convention of
// src/cuda/nvcc_src/permutate_ij_ji.cu:37-38). alpha == 0 never reads the old gradients:
// {k + 1} reads and {k} writes per element, against two read-modify-write launches per op in the
// reference (src/ops/hadamard.zig:65-79, src/ops/addition.zig:67-81).
extern "C" void launch_{name}_reverse_Scalar(
{xs}  const void* out_grads,
{gs}  double alpha,
  len_t N,
  StreamContext stream
) {{
  if (alpha == 0.0) {{
    const mp::EwPtrs<{k + 1}, {k}> ptrs{{{{{ins}, out_grads}}, {{{outs}}}}};
    mp::ew_launch<Scalar, {k + 1}, {k}, 1>(ptrs, N, {cn}ReverseOverwriteFn_Scalar{{}}, get_stream(stream));
  }} else {{
    const mp::EwPtrs<{2 * k + 1}, {k}> ptrs{{{{{ins}, out_grads, {outs}}},
                                {{{outs}}}}};
    mp::ew_launch<Scalar, {2 * k + 1}, {k}, 1>(ptrs, N, {cn}ReverseBlendFn_Scalar{{alpha}}, get_stream(stream));
  }}
}}
"""


def host_table(chains):
    """host/chains.hpp: signature -> type-erased forward / reverse calls."""
    out = [
        "// GENERATED by metaphor_amd/chaingen.py from chains.json -- do not edit.",
        "// Fused elementwise chains the host side can substitute for a pending expression. The",
        "// signature is the expression with its leaves numbered in order of first appearance.",
        "#ifndef MP_HOST_CHAINS_HPP",
        "#define MP_HOST_CHAINS_HPP",
        "",
        '#include "kernels.hpp"',
        "",
        "namespace mp {",
        "",
        "struct FusedChain {",
        "  const char* signature;",
        "  int leaves;",
        "  void (*forward)(size_t key, void* const* x, void* out, len_t n, StreamContext ctx);",
        "  void (*reverse)(size_t key, void* const* x, void* out_grads, void* const* g, double alpha, len_t n,",
        "                  StreamContext ctx);",
        "};",
        "",
    ]
    rows = []
    for c in chains:
        root, k = parse(c["expr"])
        name = c["name"]
        xs = ", ".join(f"x[{i}]" for i in range(k))
        gs = ", ".join(f"g[{i}]" for i in range(k))
        out += [
            f"inline void chain_fwd_{name}(size_t key, void* const* x, void* out, len_t n, StreamContext ctx) {{",
            f"  kernels::{name}(key, {xs}, out, n, ctx);",
            "}",
            f"inline void chain_rev_{name}(size_t key, void* const* x, void* out_grads, void* const* g, double alpha,",
            f"                          len_t n, StreamContext ctx) {{",
            f"  kernels::{name}_reverse(key, {xs}, out_grads, {gs}, alpha, n, ctx);",
            "}",
        ]
        rows.append(f'    {{"{root.signature()}", {k}, chain_fwd_{name}, chain_rev_{name}}},')
    out += ["", "inline const FusedChain fused_chains[] = {"] + rows + ["};", "",
            "}  // namespace mp", "", "#endif", ""]
    return "\n".join(out)


def zig_table(chains):
    """The same table for the Zig op layer (zig/src/ops/fused_chains.zig): one pair of functions per
    listed chain that spreads the leaf pointers into the launcher's argument list, and the table
    that src/ops/fused.zig looks a pending expression's signature up in."""
    out = [
        "// GENERATED by metaphor_amd/chaingen.py from chains.json -- do not edit.",
        "// Fused elementwise chains a pending expression can run as: its signature (leaves numbered in",
        "// order of first appearance), its leaf count, and the launchers of both directions.",
        'const core = @import("core");',
        "const StreamContext = core.utils.StreamContext;",
        "",
        "pub const Chain = struct {",
        "    signature: []const u8,",
        "    leaves: usize,",
        "    forward: *const fn (key: usize, x: []const *anyopaque, out: *anyopaque, n: usize, ctx: StreamContext) void,",
        "    reverse: *const fn (key: usize, x: []const *anyopaque, out_grads: *anyopaque, g: []const *anyopaque, alpha: f64, n: usize, ctx: StreamContext) void,",
        "};",
        "",
    ]
    rows = []
    for c in chains:
        root, k = parse(c["expr"])
        name = c["name"]
        xs = ", ".join(f"x[{i}]" for i in range(k))
        gs = ", ".join(f"g[{i}]" for i in range(k))
        out += [
            f"fn fwd_{name}(key: usize, x: []const *anyopaque, out: *anyopaque, n: usize, ctx: StreamContext) void {{",
            f"    core.invoke(core.kernels.{name}, key, .{{ {xs}, out, n, ctx }});",
            "}",
            f"fn rev_{name}(key: usize, x: []const *anyopaque, out_grads: *anyopaque, g: []const *anyopaque, alpha: f64, n: usize, ctx: StreamContext) void {{",
            f"    core.invoke(core.kernels.{name}_reverse, key, .{{ {xs}, out_grads, {gs}, alpha, n, ctx }});",
            "}",
        ]
        rows.append(f'    .{{ .signature = "{root.signature()}", .leaves = {k}, .forward = fwd_{name}, .reverse = rev_{name} }},')
    out += ["", "pub const table = [_]Chain{"] + rows + ["};", ""]
    return "\n".join(out)


def load_chains():
    with open(CHAINS) as f:
        chains = json.load(f)
    names = set()
    for c in chains:
        if not re.fullmatch(r"[a-z][a-z0-9_]*", c["name"]) or c["name"] in names:
            raise ValueError(f"bad or repeated chain name {c['name']!r}")
        names.add(c["name"])
        parse(c["expr"])
    return chains


def _write_if_changed(path, text):
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as f:
            f.write(text)
        return True
    return False


def generate():
    """Write the chain sources and the host table; returns the files that changed."""
    changed = []
    chains = load_chains()
    for c in chains:
        for path, text in ((os.path.join(SRC_DIR, c["name"] + ".hip"), forward_source(c["name"], c["expr"])),
                           (os.path.join(SRC_DIR, c["name"] + "_reverse.hip"), reverse_source(c["name"], c["expr"]))):
            if _write_if_changed(path, text):
                changed.append(path)
    if _write_if_changed(os.path.join(HOST_DIR, "chains.hpp"), host_table(chains)):
        changed.append(os.path.join(HOST_DIR, "chains.hpp"))
    if os.path.isdir(ZIG_OPS) and _write_if_changed(os.path.join(ZIG_OPS, "fused_chains.zig"), zig_table(chains)):
        changed.append(os.path.join(ZIG_OPS, "fused_chains.zig"))
    # a chain taken out of chains.json takes its generated sources with it
    wanted = {c["name"] + suffix for c in chains for suffix in (".hip", "_reverse.hip")}
    for name in sorted(os.listdir(SRC_DIR)):
        path = os.path.join(SRC_DIR, name)
        if name.endswith(".hip") and name not in wanted:
            with open(path) as f:
                if "GENERATED by metaphor_amd/chaingen.py" in f.read(400):
                    os.remove(path)
                    changed.append(path)
    return changed


if __name__ == "__main__":
    for p in generate():
        print("wrote", p)
