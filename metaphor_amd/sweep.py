"""Event-timed throughput of the launchers over shapes outside the benchmark configurations.

    python -m metaphor_amd.sweep rows         softmax / RMSNorm forward and reverse over row lengths
    python -m metaphor_amd.sweep elementwise  the elementwise launchers at 2^28 elements
    python -m metaphor_amd.sweep matrix       row / column sums, broadcasts, transpose, vector products
    python -m metaphor_amd.sweep all

Every figure is algorithmic bytes (each input read once, each output written once) divided by
the median of ten event-timed launches, in GB/s. Operands are far larger than the caches, so
nothing is served from them. Needs an MI355X; torch only owns the buffers and the events.
"""
import sys

import torch

from . import ffi
from . import workloads as W

NAME = {torch.float16: "r16", torch.float32: "r32", torch.float64: "r64"}


def _time(f, iters=10):
    f()
    f()
    torch.cuda.synchronize()
    ts = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        f()
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b))
    return sorted(ts)[len(ts) // 2]


def _rate(nbytes, ms):
    return f"{nbytes / ms / 1e6:6.0f}"


def rows(total=1 << 28):
    print("| dtype | n | m | softmax fwd | softmax rev | rmsnorm fwd | rmsnorm rev |")
    print("|---|---|---|---|---|---|---|")
    for dt in (torch.float32, torch.float16):
        es = torch.empty(0, dtype=dt).element_size()
        for n in (8, 16, 64, 256, 1000, 1024, 4096, 8192, 16384, 32768, 50257, 65536, 131072, 262144):
            m = total // n
            x = torch.randn(m, n, device="cuda", dtype=torch.float32).to(dt)
            dy = torch.randn(m, n, device="cuda", dtype=torch.float32).to(dt)
            y, dx = torch.empty_like(x), torch.empty_like(x)
            g = torch.ones(n, device="cuda", dtype=dt)
            dg = torch.empty_like(g)
            sf, sr = W.softmax_scratch(dt, m, n), W.softmax_reverse_scratch(dt, m, n)
            nf, nr = W.rmsnorm_scratch(dt, m, n), W.rmsnorm_reverse_scratch(dt, m, n)
            B = m * n * es
            t1 = _time(lambda: W.softmax_forward(x, y, sf))
            t2 = _time(lambda: W.softmax_reverse(y, dy, dx, 0.0, sr))
            t3 = _time(lambda: W.rmsnorm_forward(x, g, y, 1e-6, nf))
            t4 = _time(lambda: W.rmsnorm_reverse(x, g, dy, dx, dg, nr, 1e-6))
            print(f"| {NAME[dt]} | {n} | {m} | {_rate(2 * B, t1)} | {_rate(3 * B, t2)} | {_rate(2 * B, t3)} | "
                  f"{_rate(3 * B, t4)} |", flush=True)
            del x, y, dy, dx


def elementwise(n=1 << 28):
    print("| dtype | " + " | ".join(("addition", "hadamard", "hadamard_reverse", "relu", "selu", "selu_reverse",
                                       "dilate", "fill", "copy", "fused fwd", "fused rev")) + " |")
    print("|---|" + "---|" * 11)
    for dt in (torch.float32, torch.float16):
        es = torch.empty(0, dtype=dt).element_size()
        a, b, c, d = (torch.rand(n, device="cuda", dtype=torch.float32).mul_(4).sub_(2).to(dt) for _ in range(4))
        e = torch.empty_like(a)
        grads = [torch.empty_like(a) for _ in range(4)]
        L = lambda stem, *args: W._launch(stem, dt, *args)
        cases = [
            (3, lambda: L("addition", a.data_ptr(), b.data_ptr(), e.data_ptr(), n)),
            (3, lambda: L("hadamard", a.data_ptr(), b.data_ptr(), e.data_ptr(), n)),
            (4, lambda: L("hadamard_reverse", a.data_ptr(), b.data_ptr(), e.data_ptr(), n)),
            (2, lambda: L("relu", a.data_ptr(), e.data_ptr(), n)),
            (2, lambda: L("selu", a.data_ptr(), e.data_ptr(), n)),
            (4, lambda: L("selu_reverse", a.data_ptr(), e.data_ptr(), b.data_ptr(), n)),
            (2, lambda: L("dilate", a.data_ptr(), 0.5, e.data_ptr(), n)),
            (1, lambda: L("fill", e.data_ptr(), 0.5, n)),
            (2, lambda: L("copy", a.data_ptr(), e.data_ptr(), n)),
            (5, lambda: W.fused_forward(a, b, c, d, e)),
            (9, lambda: W.fused_reverse(a, b, c, d, e, *grads, 0.0)),
        ]
        print(f"| {NAME[dt]} | " + " | ".join(_rate(u * n * es, _time(f)) for u, f in cases) + " |", flush=True)
        del a, b, c, d, e, grads


def matrix():
    # reduce_ij_j twice: through a bare stream context (no workspace) and through one made by the library
    print("| dtype | shape | reduce_ij_i | reduce_ij_j bare | reduce_ij_j | reduce_ij_j_scratch | broadcast_i_ij | "
          "broadcast_j_ij | permutate | A.v | u.A |")
    print("|---|---|---|---|---|---|---|---|---|---|---|")
    kernels, _ = ffi.load()
    for dt in (torch.float32, torch.float16):
        es = torch.empty(0, dtype=dt).element_size()
        for (m, n) in ((16384, 16384), (262144, 1024), (1024, 262144), (65536, 4096), (20000, 50257), (1 << 24, 8), (8, 1 << 24)):
            x = (torch.randn(m, n, device="cuda") * 0.1).to(dt)
            t = torch.empty(n, m, device="cuda", dtype=dt)
            vi, vj = torch.randn(m, device="cuda").to(dt), torch.randn(n, device="cuda").to(dt)
            oi, oj = torch.empty_like(vi), torch.empty_like(vj)
            B = m * n * es
            nb = int(kernels.mpReduceScratchBytes(W.KEY[dt], m, n))
            sc = torch.empty(max(nb, 16), dtype=torch.uint8, device="cuda")
            L = lambda stem, *args: W._launch(stem, dt, *args)
            cells = [
                _rate(B, _time(lambda: L("reduce_ij_i", x.data_ptr(), oi.data_ptr(), 0.0, m, n))),
                _rate(B, _time(lambda: L("reduce_ij_j", x.data_ptr(), oj.data_ptr(), 0.0, m, n))),
                _rate(B, _time(lambda: ffi.invoke(kernels.reduce_ij_j, W.KEY[dt], x.data_ptr(), oj.data_ptr(), 0.0, m, n,
                                                  W.blas_ctx()))),
                _rate(B, _time(lambda: L("reduce_ij_j_scratch", x.data_ptr(), oj.data_ptr(),
                                         sc.data_ptr() if nb else None, 0.0, m, n))),
                _rate(B, _time(lambda: L("broadcast_i_ij", vi.data_ptr(), x.data_ptr(), 0.0, m, n))),
                _rate(B, _time(lambda: L("broadcast_j_ij", vj.data_ptr(), x.data_ptr(), 0.0, m, n))),
                _rate(2 * B, _time(lambda: W.permutate(x, t))),
                _rate(B, _time(lambda: W.inner_product("ij_jk_ik", x, vj, 1.0, oi, 0.0, m, n, 1))),
                _rate(B, _time(lambda: W.inner_product("ij_jk_ik", vi, x, 1.0, oj, 0.0, 1, m, n))),
            ]
            print(f"| {NAME[dt]} | [{m},{n}] | " + " | ".join(cells) + " |", flush=True)
            del x, t


def main(argv):
    if not torch.cuda.is_available():
        sys.exit("metaphor_amd.sweep needs a GPU")
    ffi.load()
    what = argv[1] if len(argv) > 1 else "all"
    table = {"rows": rows, "elementwise": elementwise, "matrix": matrix}
    if what != "all" and what not in table:
        sys.exit(__doc__)
    for name, fn in table.items():
        if what in ("all", name):
            print(f"\n### {name} (GB/s)\n")
            fn()


if __name__ == "__main__":
    main(sys.argv)
