"""The measurement behind the row launchers' dispatch rules: the choice the library makes for a row
length against every regime the test build can force, interleaved in one process.

    python tests/regime_ab.py r16|r32 n1,n2,...

For each row length n (operands of 2^28 elements, m = 2^28 / n rows) it times the softmax and
RMSNorm launchers, forward and reverse, under regime 0 (the library's own choice) and under the
forced groups of 128 ... 1024 threads a row and the shared-row kernels, three rounds of twelve
event-timed launches each, and prints the median rate in GB/s of algorithmic bytes with the
range over the rounds. A forced regime is starred when its median is more than 3 % above the
library's choice and its slowest round beats the choice's fastest: a candidate for a rule, to be
confirmed on a second box before it becomes one (rates move by 3-5 % from box to box; inside one
process they repeat within 1 %).

Needs an MI355X and lib/libmp_kernels_diag.so (built by `python -m metaphor_amd.kernelgen`). Not
collected by pytest. The forced launches go through the test build, the automatic ones through
the library as shipped; workspaces are sized once for the largest any regime asks for.
"""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

import numpy as np
import torch

import gpu_lib as G

NAMES = {0: "auto", 2: "G128", 3: "G256", 4: "G512", 5: "G1024", 7: "shared"}
TOTAL = 1 << 28


def timed(f, iters=12):
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
    return float(np.median(ts))


def main():
    if len(sys.argv) != 3 or sys.argv[1] not in ("r16", "r32"):
        sys.exit(__doc__)
    dt = {"r32": torch.float32, "r16": torch.float16}[sys.argv[1]]
    es = torch.empty(0, dtype=dt).element_size()
    for n in [int(a) for a in sys.argv[2].split(",")]:
        m = TOTAL // n
        x = torch.randn(m, n, device="cuda", dtype=torch.float32).to(dt)
        dy = torch.randn(m, n, device="cuda", dtype=torch.float32).to(dt)
        y, dx = torch.empty_like(x), torch.empty_like(x)
        g = torch.ones(n, device="cuda", dtype=dt)
        dg = torch.empty_like(g)
        nbytes = m * n * es
        G.set_regime(7)  # the largest workspaces any regime asks for
        big = [max(1, G.row_size(fn, dt, m, n)) for fn in G.ROW_SIZE_FNS]
        G.set_regime(0)
        sf, sr, nf, nr = (torch.empty(b, dtype=torch.uint8, device="cuda") for b in big)
        ops = {"softmax fwd": (2, lambda: G.softmax(x, y, scratch=sf)),
               "softmax rev": (3, lambda: G.softmax_reverse(y, dy, dx, 0.0, scratch=sr)),
               "rmsnorm fwd": (2, lambda: G.rmsnorm(x, g, y, 1e-6, scratch=nf)),
               "rmsnorm rev": (3, lambda: G.rmsnorm_reverse(x, g, dy, dx, dg, nr, 1e-6, 0.0))}
        rates = {(o, r): [] for o in ops for r in NAMES}
        for _ in range(3):
            for r in NAMES:
                G.set_regime(r)
                for o, (streams, f) in ops.items():
                    rates[(o, r)].append(streams * nbytes / timed(f) / 1e6)
        G.set_regime(0)
        for o in ops:
            chosen = rates[(o, 0)]
            cells = []
            for r, name in NAMES.items():
                v = rates[(o, r)]
                med = float(np.median(v))
                star = "*" if med > 1.03 * float(np.median(chosen)) and min(v) > max(chosen) else ""
                cells.append(f"{name} {med:5.0f} ({min(v):4.0f}-{max(v):4.0f}){star}")
            print(f"{sys.argv[1]} n={n:6d} {o}: " + " | ".join(cells), flush=True)
        del x, y, dy, dx


if __name__ == "__main__":
    main()
