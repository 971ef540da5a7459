"""CPU-side checks of the boundary: the libraries load, export every symbol the headers
declare, and the generator's outputs are consistent. No compute call is made."""
import ctypes
import os
import re

import pytest

from metaphor_amd import ffi, kernelgen

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_kernel_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(os.path.join(ffi.LIB_DIR, "libmp_kernels.so"))
    protos = ffi.parse_declarations()
    assert len(protos) >= 35
    for _, name, _ in protos:
        assert hasattr(lib, name), name


def test_device_utils_exports_the_eleven_reference_names():
    lib = ctypes.CDLL(os.path.join(ffi.LIB_DIR, "libdev_utils.so"))
    names = [n for _, n, _ in ffi.parse_declarations(os.path.join(ROOT, "include", "device_utils.h"))]
    reference = ["mpInitDevice", "mpMemAlloc", "mpMemcpyHtoD", "mpMemcpyDtoH", "mpMemFree",
                 "mpDeviceSynchronize", "mpStreamSynchronize", "mpInitStream", "mpDeinitStream",
                 "mpCheckLastError", "mpDeviceTotalMemory"]
    assert [n for n in names if n not in ("mpAdoptStream", "mpReleaseStream")] == reference
    assert "mpAdoptStream" in names and "mpReleaseStream" in names  # for callers that own their streams
    for n in names:
        assert hasattr(lib, n), n


def test_static_archive_holds_the_same_launchers():
    import subprocess
    out = subprocess.run(["nm", "--defined-only", os.path.join(ffi.LIB_DIR, "mp_kernels.a")],
                         capture_output=True, text=True, check=True).stdout
    defined = set(re.findall(r" T (launch_\w+|mp\w+)", out))
    for _, name, _ in ffi.parse_declarations():
        assert name in defined, name


def test_shipped_libraries_export_no_process_wide_switches():
    """Launchers must be re-entrant across streams: the regime and cluster-tuning overrides of the
    parity tests live in a library of their own, not in the shipped ones."""
    import subprocess
    for name in ("libmp_kernels.so", "mp_kernels.a"):
        flags = ["-D", "--defined-only"] if name.endswith(".so") else ["--defined-only"]
        out = subprocess.run(["nm"] + flags + [os.path.join(ffi.LIB_DIR, name)],
                             capture_output=True, text=True, check=True).stdout
        assert "mpSetRowRegime" not in out and "mpSetClusterTuning" not in out and "mpSetClusterDeep" not in out, name
        assert "mpSetClusterWords" not in out and "mpSetKeepInput" not in out and "mpDescribeRowPlans" not in out, name
        assert "row_regime_override" not in out and "cluster_tuning" not in out, name
    diag = subprocess.run(["nm", "-D", "--defined-only", os.path.join(ffi.LIB_DIR, "libmp_kernels_diag.so")],
                          capture_output=True, text=True, check=True).stdout
    assert " T mpSetRowRegime" in diag and " T mpSetClusterTuning" in diag and " T mpSetClusterDeep" in diag
    assert " T mpSetClusterWords" in diag and " T mpSetKeepInput" in diag and " T mpDescribeRowPlans" in diag


def test_dispatch_arrays_are_r16_r32_r64_in_scalar_tag_order():
    table = kernelgen.kernel_table()
    for stem, arr in table.items():
        assert arr == [f"launch_{stem}_r16", f"launch_{stem}_r32", f"launch_{stem}_r64"]
    kernels, _ = ffi.load()
    assert set(table) == set(kernels.stems())
    for stem in table:
        assert len(getattr(kernels, stem)) == 3


def test_every_launcher_takes_the_stream_context_last_and_returns_void():
    for ret, name, args in ffi.parse_declarations():
        if name.startswith("launch_"):
            assert ret == "void"
            assert args[-1][0] == "StreamContext"
            assert all(t in ("const void*", "void*", "double", "len_t") for t, _ in args[:-1])


def test_stream_context_layout_is_two_pointers_by_value():
    assert ctypes.sizeof(ffi.StreamContext) == 16
    assert ffi.StreamContext.hip_stream.offset == 0 and ffi.StreamContext.blas_handle.offset == 8


def test_generated_header_is_current():
    before = open(kernelgen.DECLS).read()
    kernelgen.make_kernel_declarations()
    assert open(kernelgen.DECLS).read() == before


def test_config_rejects_non_gfx_architectures(tmp_path, monkeypatch):
    cfg = tmp_path / "config.json"
    cfg.write_text('{"gpu-architecture": "sm_89"}')
    monkeypatch.setattr(kernelgen, "CONFIG", str(cfg))
    with pytest.raises(ValueError):
        kernelgen.load_config()


def test_headers_compile_as_plain_c_and_link(tmp_path):
    """The boundary is a C ABI: a C11 translation unit includes the three headers, takes the
    address of a launcher and of a device utility, and links against the two libraries (nothing
    is called: there is no GPU here)."""
    import subprocess
    src = tmp_path / "abi.c"
    src.write_text(
        '#include "tensor_types.h"\n#include "device_utils.h"\n#include "kernel_decls.h"\n'
        "typedef void (*softmax_fn)(const void*, void*, void*, len_t, len_t, StreamContext);\n"
        "typedef StreamContext (*init_fn)(void);\n"
        "int main(void) {\n"
        "  softmax_fn f = launch_softmax_ij_j_r32;\n"
        "  init_fn g = mpInitStream;\n"
        "  StreamContext c; c.hip_stream.ptr = 0; c.blas_handle.ptr = 0;\n"
        "  return (f != 0 && g != 0 && sizeof c == 2 * sizeof(void*) && sizeof(r16) == 2) ? 0 : 1;\n"
        "}\n")
    exe = tmp_path / "abi"
    cmd = ["gcc", "-std=c11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
           "-L", ffi.LIB_DIR, "-lmp_kernels", "-ldev_utils", f"-Wl,-rpath,{ffi.LIB_DIR}", "-Wl,-rpath-link,/opt/rocm/lib"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
