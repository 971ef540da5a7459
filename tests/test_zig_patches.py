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


OP_MODULES = ("selu.zig", "softmax.zig", "rmsnorm.zig", "fused.zig", "fused_chains.zig")


def test_op_modules_call_only_what_the_boundary_declares():
    decls = open(os.path.join(ROOT, "include", "kernel_decls.h")).read()
    stems = set(re.findall(r"launch_(\w+)_r32\(", decls))
    sizes = set(re.findall(r"len_t (mp\w+ScratchBytes)\(", decls))
    for mod in OP_MODULES:
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
    for mod in OP_MODULES:
        text = open(os.path.join(ZIG, "src", "ops", mod)).read()
        for m in re.finditer(r"core\.invoke\(core\.kernels\.(\w+),\s*[\w.()]+,\s*\.\{(.*?)\}\s*\)", text, re.S):
            args = [a for a in re.sub(r"@as\([^)]*\)|\([^()]*\)", "X", m.group(2)).split(",") if a.strip()]
            assert len(args) == arity[m.group(1)], (mod, m.group(1), len(args), arity[m.group(1)])


def test_the_generated_chain_table_is_current_and_matches_the_host_table():
    from metaphor_amd import chaingen
    chains = chaingen.load_chains()
    assert open(os.path.join(ZIG, "src", "ops", "fused_chains.zig")).read() == chaingen.zig_table(chains)
    zig_rows = re.findall(r'\.signature = "([^"]+)", \.leaves = (\d+)', chaingen.zig_table(chains))
    cpp_rows = re.findall(r'\{"([^"]+)", (\d+), chain_fwd', chaingen.host_table(chains))
    assert zig_rows == cpp_rows and len(zig_rows) == len(chains)


def test_the_fusion_bindings_match_the_header():
    """The extern fn lines of fused.zig take as many parameters as include/chain_fusion.h declares."""
    header = open(os.path.join(ROOT, "include", "chain_fusion.h")).read()
    want = {m.group(1): len([a for a in m.group(2).split(",") if a.strip() and a.strip() != "void"])
            for m in re.finditer(r"EXTERN_C [\w ]+?\*?\s*(mpChain\w+)\(([^)]*)\)", header)}
    text = open(os.path.join(ZIG, "src", "ops", "fused.zig")).read()
    got = {m.group(1): len([a for a in m.group(2).split(",") if a.strip()])
           for m in re.finditer(r"extern fn (mpChain\w+)\(([^)]*)\)", text)}
    assert got and set(got) <= set(want)
    for name, count in got.items():
        assert count == want[name], (name, count, want[name])


def _quoted_includes(path):
    return re.findall(r'^\s*#\s*include\s+"([^"]+)"', open(path).read(), re.M)


@pytest.mark.skipif(not os.path.isdir(REFERENCE) or shutil.which("patch") is None,
                    reason="needs the reference tree and patch(1); neither travels to the GPU box")
def test_the_patched_tree_finds_every_file_it_opens(tmp_path):
    """All patches applied to a scratch copy of the files they touch, the shipped sources laid out as
    zig/README.md says, then a walk over what the patched build would open: the kernel sources, the
    files behind append_kernel_directory() in build.zig and file_gen.zig (device_utils and the
    headers that cimport.zig @cIncludes), every quoted #include of the device sources, and every
    @import of an op module."""
    tree = tmp_path / "tree"
    for name in PATCHES:
        text = open(os.path.join(ZIG, "patches", name)).read()
        target = re.search(r"^\+\+\+ b/(\S+)", text, re.M).group(1)
        dst = tree / target
        dst.parent.mkdir(parents=True, exist_ok=True)
        if not dst.exists():
            shutil.copy(os.path.join(REFERENCE, target), dst)
        res = subprocess.run(["patch", "-p1", "--no-backup-if-mismatch", "-i", os.path.join(ZIG, "patches", name)],
                             cwd=tree, capture_output=True, text=True)
        assert res.returncode == 0, name + res.stdout + res.stderr
    # the reference's own op modules stay where they are (read-only: only their names are needed)
    ref_ops = set(os.listdir(os.path.join(REFERENCE, "src", "ops")))
    # the layout of zig/README.md
    csrc = os.path.join(ROOT, "metaphor_amd", "csrc")
    hip = tree / "src" / "hip"
    (hip / "hipcc_src").mkdir(parents=True)
    for f in os.listdir(csrc):
        if f.endswith(".h") or f in ("device_utils.hip", "kernel_support.hip", "noalloc_entry.hip"):
            shutil.copy(os.path.join(csrc, f), hip / f)
    for f in ("tensor_types.h", "device_utils.h"):
        shutil.copy(os.path.join(ROOT, "include", f), hip / f)
    for f in os.listdir(os.path.join(csrc, "hipcc_src")):
        shutil.copy(os.path.join(csrc, "hipcc_src", f), hip / "hipcc_src" / f)
    for f in os.listdir(os.path.join(ZIG, "src", "ops")):
        shutil.copy(os.path.join(ZIG, "src", "ops", f), tree / "src" / "ops" / f)

    build = (tree / "build.zig").read_text()
    gen = (tree / "file_gen.zig").read_text()
    fields = dict(re.findall(r"\.(source_directory|target_directory) = b\.pathJoin\(&\.\{ ([^}]*) \}\)", build))
    source_dir = os.path.join(*re.findall(r'"([^"]+)"', fields["source_directory"]))
    ext = re.search(r'\.source_extension = "([^"]+)"', build).group(1)
    assert (source_dir, ext) == (os.path.join("src", "hip", "hipcc_src"), ".hip")
    sources = [f for f in os.listdir(tree / source_dir) if f.endswith(ext)]
    assert len(sources) >= 40 and all("Scalar" in (tree / source_dir / f).read_text() for f in sources)
    # file_gen.zig: the device directory is the parent of the configured source directory
    body = re.search(r"pub fn append_kernel_directory\(.*?\n\}", gen, re.S).group(0)
    assert "std.fs.path.dirname(self.source_directory)" in body and '"cuda"' not in body
    device_dir = os.path.dirname(source_dir)
    generated = {"kernel_decls.h"}  # written there by make_kernel_declarations before anything reads it
    wanted = set(re.findall(r'append_kernel_directory\("([^"]+)"\)', build + gen))
    assert {"device_utils.hip", "device_utils.h", "tensor_types.h", "kernel_decls.h"} <= wanted
    for name in wanted - generated:
        assert (tree / device_dir / name).exists(), f"the patched build opens {device_dir}/{name}, which the layout does not provide"
    # nothing of the CUDA tree is named any more by the three build files
    for f in ("build.zig", "file_gen.zig", "script_compiler.zig"):
        code = "\n".join(l.split("//")[0] for l in (tree / f).read_text().splitlines())
        assert not re.search(r'"cuda"|nvcc|cublas|cudart|"sm_', code), f
    # every quoted include of the device sources resolves from the file that names it
    for base, _, files in os.walk(hip):
        for f in files:
            for inc in _quoted_includes(os.path.join(base, f)):
                if os.path.basename(inc) in generated:
                    continue
                assert os.path.exists(os.path.normpath(os.path.join(base, inc))), f"{f} includes {inc}"
    # every op module that src/metaphor.zig or another op module imports exists
    have = ref_ops | set(os.listdir(tree / "src" / "ops"))
    for name in re.findall(r'@import\("ops/(\w+\.zig)"\)', (tree / "src" / "metaphor.zig").read_text()):
        assert name in have, name
    for f in os.listdir(os.path.join(ZIG, "src", "ops")):
        for name in re.findall(r'@import\("(\w+\.zig)"\)', (tree / "src" / "ops" / f).read_text()):
            assert name in have, (f, name)
    # the libraries the patched build links are the ones this repository builds or ROCm ships
    assert set(re.findall(r'linkSystemLibrary\("(\w+)"\)', build)) == {"amdhip64", "dev_utils", "mp_fusion", "rocblas"}
