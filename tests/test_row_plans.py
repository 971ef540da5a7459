"""The dispatch of the four row launchers, swept on the CPU: the test build of the library runs each
launcher's whole decision on a dry run (no launch, a made-up compute-unit count, made-up operand
addresses) and reports the kernel it would enqueue. For every row length from 1 to 300 000, every
storage type, forward and reverse, GPUs of 64, 256 and 304 compute units and operands aligned,
shifted alike and shifted apart: a kernel is chosen; its workgroup is 64 ... 1024 threads in whole
wavefronts; the threads that hold a row, times the packs a thread holds, cover the row; the packs a
thread holds fit the registers that kernel family is written for; no more workgroups are launched
than there are rows to give them; and the bytes of workspace the launch may touch never exceed
what the workspace-size function of the same library asks the caller for."""
import ctypes
import os

import numpy as np
import pytest

from metaphor_amd import ffi

SHORT, RESIDENT, PAIRED, ANY, CLUSTER, DEEP, STREAM, LOOSE = range(8)
KIND, GROUP, PPT, RPB, GRID, BLOCK, PER_ROW, CHUNK, WORKSPACE, KEPT = range(10)
OPS = {"softmax": 0, "softmax_reverse": 1, "rmsnorm": 2, "rmsnorm_reverse": 3}
ELEM = {0: 2, 1: 4, 2: 8}            # bytes of r16, r32, r64
ACC = {0: 4, 1: 4, 2: 8}             # bytes of precision<T>
# 32-bit registers a thread may spend on ONE row-shaped array of widened values in each family
# (row_dispatch.h: max_nv_for; the shared-row kernels keep r16 chunks in their storage type)
REGISTERS = {0: 64, 1: 32, 2: 32, 3: 16}
N_HI = 300001


def _lib():
    path = os.path.join(ffi.LIB_DIR, "libmp_kernels_diag.so")
    if not os.path.exists(path):
        raise ffi.BoundaryMissing(f"{path} is not built; run `python -m metaphor_amd.kernelgen`")
    d = ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)
    d.mpDescribeRowPlans.argtypes = [ctypes.c_ulong] * 7 + [ctypes.c_void_p, ctypes.c_void_p]
    d.mpDescribeRowPlans.restype = ctypes.c_ulong
    return d


def _plans(lib, op, dtype, m, cus, shift):
    notes = np.zeros((N_HI - 1, 10), dtype=np.int64)
    sizes = np.zeros(N_HI - 1, dtype=np.uint64)
    noted = lib.mpDescribeRowPlans(op, dtype, m, 1, N_HI, cus, shift, notes.ctypes.data, sizes.ctypes.data)
    return int(noted), notes, sizes.astype(np.int64)


CASES = [(cus, m, 0) for cus in (64, 256, 304) for m in (1, 8192)] + [(256, 8192, 1), (256, 8192, 2), (256, 3, 1)]


@pytest.mark.parametrize("dtype", [0, 1, 2], ids=["r16", "r32", "r64"])
@pytest.mark.parametrize("op", sorted(OPS), ids=sorted(OPS))
def test_every_row_length_gets_a_kernel_that_holds_it(op, dtype):
    lib = _lib()
    w = 16 // ELEM[dtype]
    n = np.arange(1, N_HI, dtype=np.int64)
    packs = (n + w - 1) // w
    for cus, m, shift in CASES:
        what = f"{op} dtype {dtype} m {m} cus {cus} shift {shift}"
        noted, p, size = _plans(lib, OPS[op], dtype, m, cus, shift)
        assert noted == N_HI - 1, f"{what}: {N_HI - 1 - noted} row lengths without a kernel"
        kind = p[:, KIND]
        assert ((kind >= SHORT) & (kind <= LOOSE)).all(), what
        assert ((p[:, BLOCK] % 64 == 0) & (p[:, BLOCK] >= 64) & (p[:, BLOCK] <= 1024)).all(), what
        assert ((p[:, GRID] >= 1) & (p[:, GRID] < 2 ** 31)).all(), what

        held = np.isin(kind, (RESIDENT, PAIRED, ANY, LOOSE))
        bad = held & (p[:, GROUP] * p[:, PPT] < packs)
        assert not bad.any(), f"{what}: n = {n[bad][:5]} not covered by group x packs a thread"
        short = kind == SHORT
        assert not (short & ((p[:, GROUP] < packs) | (packs > 16))).any(), what
        shared = np.isin(kind, (CLUSTER, DEEP))
        bad = shared & ((p[:, PER_ROW] * p[:, CHUNK] < packs) | (p[:, CHUNK] > 1024 * p[:, PPT]) | (p[:, PER_ROW] > 64))
        assert not bad.any(), f"{what}: n = {n[bad][:5]}: the chunks of a shared row do not cover it or exceed the register tile"
        # rows in groups: the groups of a workgroup fill it, and no workgroup is launched without a row
        grouped = held | short
        assert not (grouped & (p[:, GROUP] * p[:, RPB] > p[:, BLOCK])).any(), what
        assert not (grouped & (p[:, GRID] > (m + p[:, RPB] - 1) // p[:, RPB])).any(), what
        assert not (shared & (p[:, GRID] > m * p[:, PER_ROW])).any(), what
        assert not ((kind == STREAM) & (p[:, GRID] > max(m, 1))).any(), what
        # persistent grids stay within two workgroups a compute unit
        persistent = np.isin(kind, (PAIRED, ANY, STREAM, DEEP)) | ((kind == RESIDENT) & (OPS[op] >= 2) & (p[:, BLOCK] == 1024))
        assert not (persistent & (p[:, GRID] > 2 * cus)).any(), what

        per_pack = w * (ACC[dtype] // 4)
        raw = shared | ((kind == ANY) & (dtype == 0))  # r16 kept as loaded: four registers a pack
        regs = np.where(raw, p[:, PPT] * 4, p[:, PPT] * per_pack)
        bad = (held | shared) & (regs > REGISTERS[OPS[op]])
        assert not bad.any(), f"{what}: n = {n[bad][:5]} held at {p[bad][:5, PPT]} packs a thread"

        bad = p[:, WORKSPACE] > size
        assert not bad.any(), (f"{what}: n = {n[bad][:5]} may touch {p[bad][:5, WORKSPACE]} bytes of a workspace "
                               f"sized {size[bad][:5]}")


def test_the_benchmark_shapes_take_the_kernels_the_design_names():
    """cfg1 / cfg3: one-shot groups of 128 threads at two packs; cfg2: 1024 threads a row at one pack,
    rows in pairs in reverse, one workgroup a compute unit; cfg5a / cfg5b: rows shared by 8 and 3
    workgroups (reverse: 10 and 4)."""
    lib = _lib()

    def one(op, dtype, m, n, cus=256):
        notes = np.zeros((1, 10), dtype=np.int64)
        sizes = np.zeros(1, dtype=np.uint64)
        assert lib.mpDescribeRowPlans(OPS[op], dtype, m, n, n + 1, cus, 0, notes.ctypes.data, sizes.ctypes.data) == 1
        return notes[0], int(sizes[0])

    p, _ = one("softmax", 1, 256, 1024)
    assert (p[KIND], p[GROUP], p[PPT]) == (RESIDENT, 128, 2)
    p, _ = one("softmax", 0, 524288, 2048)
    assert (p[KIND], p[GROUP], p[PPT]) == (RESIDENT, 128, 2)
    p, _ = one("rmsnorm", 1, 8192, 4096)
    assert (p[KIND], p[GROUP], p[PPT], p[GRID]) == (RESIDENT, 1024, 1, 512)
    p, size = one("rmsnorm_reverse", 1, 8192, 4096)
    assert (p[KIND], p[GROUP], p[PPT], p[GRID]) == (PAIRED, 1024, 1, 256)
    assert p[WORKSPACE] == 256 * 4096 * 4 and size >= p[WORKSPACE]
    for (m, n), fwd, rev in (((512, 151936), 8, 10), ((2048, 50257), 3, 4)):
        p, size = one("softmax", 1, m, n)
        assert (p[KIND], p[PER_ROW]) == (CLUSTER, fwd) and p[GRID] == m * fwd and 0 < p[WORKSPACE] <= size
        p, size = one("softmax_reverse", 1, m, n)
        assert (p[KIND], p[PER_ROW]) == (CLUSTER, rev) and 0 < p[WORKSPACE] <= size


@pytest.mark.parametrize("dtype", [0, 1], ids=["r16", "r32"])
def test_forwards_keep_a_tensor_for_their_reverse_by_its_size(dtype):
    """The RMSNorm forward leaves an input of up to 256 MiB, the softmax forward an output of up to
    128 MiB, in the memory-side cache (its kernels' KEEP variants), larger tensors stream past it;
    only the kernels for aligned rows of whole packs have the variant, and no reverse has one."""
    lib = _lib()
    w = 16 // ELEM[dtype]
    n = np.arange(1, N_HI, dtype=np.int64)
    whole = n % w == 0
    for m in (64, 512, 4096, 32768):
        nbytes = m * n * ELEM[dtype]
        _, p, _ = _plans(lib, OPS["rmsnorm"], dtype, m, 256, 0)
        able = np.isin(p[:, KIND], (RESIDENT, ANY)) & whole
        want = able & (nbytes <= 256 << 20)
        assert (p[:, KEPT] == want).all(), f"rmsnorm m {m}: n = {n[p[:, KEPT] != want][:5]}"
        assert want.any() or m * N_HI * ELEM[dtype] < (256 << 20) or not able.any()
        _, p, _ = _plans(lib, OPS["softmax"], dtype, m, 256, 0)
        able = ((p[:, KIND] == RESIDENT) & whole) | (p[:, KIND] == CLUSTER)
        want = able & (nbytes <= 128 << 20)
        assert (p[:, KEPT] == want).all(), f"softmax m {m}: n = {n[p[:, KEPT] != want][:5]}"
        for op in ("softmax_reverse", "rmsnorm_reverse"):
            _, p, _ = _plans(lib, OPS[op], dtype, m, 256, 0)
            assert not p[:, KEPT].any(), f"{op} m {m}"
    # operands shifted off their 16-byte alignment: no variant keeps anything but the shared-row softmax
    _, p, _ = _plans(lib, OPS["rmsnorm"], dtype, 512, 256, 1)
    assert not p[:, KEPT].any()
