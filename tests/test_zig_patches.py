"""The Zig side of the re-targeting is shipped as patches against the reference tree. No Zig
toolchain exists here, so the patched files cannot be compiled; what can be checked is that every
hunk still applies to the reference it was cut from, and that the new op modules only call
launchers and size functions that the boundary headers declare."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ZIG = os.path.join(ROOT, "zig")
REFERENCE = "/root/reference"

PATCHES = sorted(f for f in os.listdir(os.path.join(ZIG, "patches")) if f.endswith(".patch"))


@pytest.mark.skipif(not os.path.isdir(REFERENCE) or shutil.which("patch") is None,
                    reason="needs the reference tree and patch(1); neither travels to the GPU box")
@pytest.mark.parametrize("name", PATCHES)
def test_patch_applies_to_the_reference_it_was_cut_from(name, tmp_path):
    text = open(os.path.join(ZIG, "patches", name)).read()
    target = re.search(r"^\+\+\+ b/(\S+)", text, re.M).group(1)
    dst = tmp_path / target
    dst.parent.mkdir(parents=True, exist_ok=True)
    shutil.copy(os.path.join(REFERENCE, target), dst)  # a copy in a scratch directory: the reference is never written
    res = subprocess.run(["patch", "-p1", "--no-backup-if-mismatch", "-i", os.path.join(ZIG, "patches", name)],
                         cwd=tmp_path, capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "fuzz" not in res.stdout and "offset" not in res.stdout, res.stdout
    assert not list(tmp_path.rglob("*.rej"))


def test_op_modules_call_only_what_the_boundary_declares():
    decls = open(os.path.join(ROOT, "include", "kernel_decls.h")).read()
    stems = set(re.findall(r"launch_(\w+)_r32\(", decls))
    sizes = set(re.findall(r"len_t (mp\w+ScratchBytes)\(", decls))
    for mod in ("selu.zig", "softmax.zig", "rmsnorm.zig"):
        text = open(os.path.join(ZIG, "src", "ops", mod)).read()
        used = set(re.findall(r"core\.kernels\.(\w+)", text))
        assert used and used <= stems, (mod, used - stems)
        assert set(re.findall(r"dev\.(mp\w+)", text)) <= sizes, mod
    patch = open(os.path.join(ZIG, "patches", "src_ops_inner_product.zig.patch")).read()
    added = set(re.findall(r"^\+.*core\.kernels\.(\w+)", patch, re.M))
    assert added and added <= stems, added


def test_launcher_argument_counts_match_the_headers():
    """Each core.invoke(core.kernels.<stem>, key, .{ ... }) in the op modules passes as many
    arguments as launch_<stem>_r32 takes."""
    decls = open(os.path.join(ROOT, "include", "kernel_decls.h")).read()
    arity = {m.group(1): len([a for a in m.group(2).split(",") if a.strip()])
             for m in re.finditer(r"launch_(\w+)_r32\(([^)]*)\)", decls)}
    for mod in ("selu.zig", "softmax.zig", "rmsnorm.zig"):
        text = open(os.path.join(ZIG, "src", "ops", mod)).read()
        for m in re.finditer(r"core\.invoke\(core\.kernels\.(\w+),\s*[\w.()]+,\s*\.\{(.*?)\}\s*\)", text, re.S):
            args = [a for a in re.sub(r"@as\([^)]*\)|\([^()]*\)", "X", m.group(2)).split(",") if a.strip()]
            assert len(args) == arity[m.group(1)], (mod, m.group(1), len(args), arity[m.group(1)])
