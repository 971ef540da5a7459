import os
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (_ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """Tests load what is built; only when nothing is built (a fresh checkout) build it once."""
    from metaphor_amd import ffi, kernelgen
    needed = ("libmp_kernels.so", "libdev_utils.so", "mp_kernels.a", "libmetaphor_host.so", "host_check")
    if not all(os.path.exists(os.path.join(ffi.LIB_DIR, n)) for n in needed):
        kernelgen.build(verbose=True)
