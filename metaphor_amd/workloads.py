"""The seeded synthetic workloads this path is measured and checked on, and thin Python
wrappers that enqueue the launchers of the C-ABI on torch-owned device memory.

torch is plumbing here (device buffers, the current stream, the seeded generators); every
computation is one of the ``launch_*`` entry points of include/kernel_decls.h.

Workloads (N(mu, s) = mean mu, standard deviation s; seed 0 unless a set index is added):
  cfg1  softmax forward, r32, [256, 1024], inputs 4*N(0,1)
  cfg2  RMSNorm forward + reverse, r32, X and dY [8192, 4096] ~ N(0,1), gain ~ N(1, 0.02), eps 1e-6
  cfg3  softmax forward + reverse, r16, [8*32*2048, 2048] ~ N(0,2) with -inf strictly above the
        diagonal of every 2048-row block, dY ~ N(0,1)
  cfg4  fused e = selu((a+b)*(c+d)) forward + reverse, r32, flat 2^28, inputs U(-2,2), de ~ N(0,1)
  cfg5a softmax forward, r32, [512, 151936], N(0,3) + 12 on one random column per row
  cfg5b softmax forward, r32, [2048, 50257], same distribution
  permutate  transpose, r32, [16384, 16384] ~ N(0,1); reverse = the accumulating transpose (alpha 1)
  gemm       c = a.b, r16 with fp32 accumulation, [8192, 8192] x [8192, 8192], inputs N(0, 0.25);
             reverse = the two products of its gradient (G.T(b) and T(a).G)
"""
import torch

from . import ffi

KEY = {torch.float16: ffi.R16, torch.float32: ffi.R32, torch.float64: ffi.R64}
DTYPE_NAME = {torch.float16: "r16", torch.float32: "r32", torch.float64: "r64"}


_contexts = {}   # stream handle -> StreamContext (a launch-bound workload pays for every object it makes)
_launchers = {}  # (stem, dtype) -> the C function


def _ctx():
    handle = torch.cuda.current_stream().cuda_stream
    ctx = _contexts.get(handle)
    if ctx is None:
        ctx = _contexts[handle] = ffi.StreamContext.from_handle(handle)
    return ctx


def _launch(stem, dtype, *args):
    fn = _launchers.get((stem, dtype))
    if fn is None:
        kernels, _ = ffi.load()
        fn = _launchers[(stem, dtype)] = getattr(kernels, stem)[KEY[dtype]]
    fn(*args, _ctx())


_blas_contexts = {}


def blas_ctx():
    """Context of torch's current stream carrying a rocBLAS handle (made once per stream)."""
    _, utils = ffi.load()
    handle = torch.cuda.current_stream().cuda_stream
    if handle not in _blas_contexts:
        _blas_contexts[handle] = utils.mpAdoptStream(handle or None)
    return _blas_contexts[handle]


# ------------------------------------------------------------------ launch wrappers

def _workspace(scratch, size_fn, dtype, m, n, what):
    """Pointer of a caller-owned workspace after checking that it is large enough for THIS dtype
    and shape: a workspace sized for another dtype would be overrun on the GPU."""
    if scratch is None:
        return None
    kernels, _ = ffi.load()
    need = int(getattr(kernels, size_fn)(KEY[dtype], m, n))
    have = scratch.numel() * scratch.element_size()
    if have < need:
        raise ValueError(f"{what}: workspace of {have} bytes, {need} needed for {DTYPE_NAME[dtype]} [{m},{n}]")
    return scratch.data_ptr()


def permutate(src, dst, alpha=0.0):
    rows, cols = src.shape
    _launch("permutate_ij_ji", src.dtype, src.data_ptr(), dst.data_ptr(), float(alpha), rows, cols)


def inner_product(form, a, b, alpha, c, beta, m, n, k):
    """form "ij_jk_ik", "ij_kj_ik" or "ji_jk_ik": c[m,k] = alpha * op(a).op(b) + beta * c over n."""
    kernels, _ = ffi.load()
    ffi.invoke(getattr(kernels, "inner_product_" + form), KEY[a.dtype], a.data_ptr(), b.data_ptr(),
               float(alpha), c.data_ptr(), float(beta), m, n, k, blas_ctx())


def softmax_scratch(dtype, m, n):
    """Workspace for launch_softmax_ij_j (None when the rows fit one workgroup)."""
    kernels, _ = ffi.load()
    nbytes = int(kernels.mpSoftmaxScratchBytes(KEY[dtype], m, n))
    return torch.empty(nbytes, dtype=torch.uint8, device="cuda") if nbytes else None


def softmax_forward(x, y, scratch=None):
    m, n = x.shape
    _launch("softmax_ij_j", x.dtype, x.data_ptr(), y.data_ptr(),
            _workspace(scratch, "mpSoftmaxScratchBytes", x.dtype, m, n, "softmax_forward"), m, n)


def softmax_reverse_scratch(dtype, m, n):
    """Workspace for launch_softmax_ij_j_reverse (None when the rows fit one workgroup)."""
    kernels, _ = ffi.load()
    nbytes = int(kernels.mpSoftmaxReverseScratchBytes(KEY[dtype], m, n))
    return torch.empty(nbytes, dtype=torch.uint8, device="cuda") if nbytes else None


def softmax_reverse(y, dy, dx, alpha=0.0, scratch=None):
    m, n = y.shape
    _launch("softmax_ij_j_reverse", y.dtype, y.data_ptr(), dy.data_ptr(), dx.data_ptr(),
            _workspace(scratch, "mpSoftmaxReverseScratchBytes", y.dtype, m, n, "softmax_reverse"), float(alpha), m, n)


def rmsnorm_scratch(dtype, m, n):
    """Workspace for launch_rmsnorm_ij_j (None when the rows fit one workgroup)."""
    kernels, _ = ffi.load()
    nbytes = int(kernels.mpRmsnormScratchBytes(KEY[dtype], m, n))
    return torch.empty(nbytes, dtype=torch.uint8, device="cuda") if nbytes else None


def rmsnorm_forward(x, gain, y, eps, scratch=None):
    m, n = x.shape
    _launch("rmsnorm_ij_j", x.dtype, x.data_ptr(), gain.data_ptr(), y.data_ptr(),
            _workspace(scratch, "mpRmsnormScratchBytes", x.dtype, m, n, "rmsnorm_forward"), float(eps), m, n)


def rmsnorm_reverse_scratch(dtype, m, n):
    kernels, _ = ffi.load()
    nbytes = int(kernels.mpRmsnormReverseScratchBytes(KEY[dtype], m, n))
    return torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")


def rmsnorm_reverse(x, gain, dy, dx, dgain, scratch, eps, alpha=0.0):
    m, n = x.shape
    _launch("rmsnorm_ij_j_reverse", x.dtype, x.data_ptr(), gain.data_ptr(), dy.data_ptr(), dx.data_ptr(),
            dgain.data_ptr(), _workspace(scratch, "mpRmsnormReverseScratchBytes", x.dtype, m, n, "rmsnorm_reverse"),
            float(eps), float(alpha), m, n)


def fused_forward(a, b, c, d, e):
    _launch("fused_selu_hadamard_add_add", a.dtype, a.data_ptr(), b.data_ptr(), c.data_ptr(),
            d.data_ptr(), e.data_ptr(), a.numel())


def fused_reverse(a, b, c, d, de, da, db, dc, dd, alpha=0.0):
    _launch("fused_selu_hadamard_add_add_reverse", a.dtype, a.data_ptr(), b.data_ptr(), c.data_ptr(),
            d.data_ptr(), de.data_ptr(), da.data_ptr(), db.data_ptr(), dc.data_ptr(), dd.data_ptr(),
            float(alpha), a.numel())


# ------------------------------------------------------------------ workload definitions

def _gen(seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return g


class Workload:
    """One buffer set of one config. `forward()` / `reverse()` enqueue the launchers;
    `fwd_bytes` / `rev_bytes` are the algorithmic HBM bytes of one call (each input read once,
    each output written once); `rows` is rows (elements for cfg4) per call."""
    name = ""
    dtype = torch.float32
    has_reverse = True
    # (streams read, streams written) by one forward / reverse call; every stream has
    # fwd_bytes / (reads + writes) bytes. bench.py times a plain pass with the same mix beside it.
    fwd_mix, rev_mix = (1, 1), (2, 1)

    def forward(self):
        raise NotImplementedError

    def reverse(self):
        raise NotImplementedError


class Cfg1(Workload):
    name, dtype, has_reverse = "cfg1", torch.float32, False
    shape = (256, 1024)

    def __init__(self, seed=0, shape=None):
        self.shape = shape or self.shape
        g = _gen(seed)
        self.x = 4.0 * torch.randn(self.shape, generator=g, device="cuda", dtype=torch.float32)
        self.y = torch.empty_like(self.x)
        self.rows = self.shape[0]
        self.fwd_bytes = 2 * self.x.numel() * 4
        self.rev_bytes = 0

    def forward(self):
        softmax_forward(self.x, self.y)


class Cfg2(Workload):
    name, dtype = "cfg2", torch.float32
    shape = (8192, 4096)
    eps = 1e-6

    def __init__(self, seed=0, shape=None):
        self.shape = shape or self.shape
        m, n = self.shape
        g = _gen(seed)
        self.x = torch.randn(self.shape, generator=g, device="cuda", dtype=torch.float32)
        self.gain = 1.0 + 0.02 * torch.randn((n,), generator=g, device="cuda", dtype=torch.float32)
        self.dy = torch.randn(self.shape, generator=g, device="cuda", dtype=torch.float32)
        self.y = torch.empty_like(self.x)
        self.dx = torch.empty_like(self.x)
        self.dgain = torch.empty_like(self.gain)
        self.scratch = rmsnorm_reverse_scratch(torch.float32, m, n)
        self.rows = m
        self.fwd_bytes = 2 * m * n * 4
        self.rev_bytes = 3 * m * n * 4

    def forward(self):
        rmsnorm_forward(self.x, self.gain, self.y, self.eps)

    def reverse(self):
        rmsnorm_reverse(self.x, self.gain, self.dy, self.dx, self.dgain, self.scratch, self.eps, 0.0)


class Cfg3(Workload):
    name, dtype = "cfg3", torch.float16
    shape = (8 * 32 * 2048, 2048)
    block = 2048

    def __init__(self, seed=0, shape=None, block=None):
        self.shape = shape or self.shape
        self.block = block or self.block
        m, n = self.shape
        g = _gen(seed)
        self.x = torch.empty(self.shape, device="cuda", dtype=torch.float16)
        self.dy = torch.empty(self.shape, device="cuda", dtype=torch.float16)
        cols = torch.arange(n, device="cuda").view(1, n)
        step = min(m, 1 << 15)
        for lo in range(0, m, step):  # chunked so the fp32 staging stays small
            hi = min(m, lo + step)
            t = 2.0 * torch.randn((hi - lo, n), generator=g, device="cuda", dtype=torch.float32)
            rows = (torch.arange(lo, hi, device="cuda") % self.block).view(-1, 1)
            t.masked_fill_(cols > rows, float("-inf"))
            self.x[lo:hi] = t.to(torch.float16)
            self.dy[lo:hi] = torch.randn((hi - lo, n), generator=g, device="cuda", dtype=torch.float32).to(torch.float16)
        self.y = torch.empty_like(self.x)
        self.dx = torch.empty_like(self.x)
        self.rows = m
        self.fwd_bytes = 2 * m * n * 2
        self.rev_bytes = 3 * m * n * 2

    def forward(self):
        softmax_forward(self.x, self.y)

    def reverse(self):
        # consumes the forward output of this set
        softmax_reverse(self.y, self.dy, self.dx, 0.0)


class Cfg4(Workload):
    name, dtype = "cfg4", torch.float32
    n = 1 << 28
    fwd_mix, rev_mix = (4, 1), (5, 4)

    def __init__(self, seed=0, n=None):
        self.n = n or self.n
        g = _gen(seed)

        def unif():
            return torch.rand((self.n,), generator=g, device="cuda", dtype=torch.float32).mul_(4.0).sub_(2.0)

        self.a, self.b, self.c, self.d = unif(), unif(), unif(), unif()
        self.de = torch.randn((self.n,), generator=g, device="cuda", dtype=torch.float32)
        self.e = torch.empty_like(self.a)
        self.da, self.db, self.dc, self.dd = (torch.empty_like(self.a) for _ in range(4))
        self.rows = self.n
        self.fwd_bytes = 20 * self.n
        self.rev_bytes = 36 * self.n

    def forward(self):
        fused_forward(self.a, self.b, self.c, self.d, self.e)

    def reverse(self):
        fused_reverse(self.a, self.b, self.c, self.d, self.de, self.da, self.db, self.dc, self.dd, 0.0)


class Cfg4Mid(Cfg4):
    """cfg4's chain on tensors of 32 MiB: inputs that together fit the memory-side cache, which the
    forward therefore leaves there for its reverse (not a BASELINE configuration)."""
    name = "cfg4mid"
    n = 1 << 23


class RuntimeChain(Cfg4):
    """cfg4's size and stream mix (4 reads + 1 write forward, 5 + 4 reverse) for an expression no
    build listed: relu((a - b) * (c + d)) is compiled by the fusion library on first use."""
    name = "chain"
    expr = b"relu(mul(sub(0,1),add(2,3)))"

    def __init__(self, seed=0, n=None):
        import ctypes
        super().__init__(seed, n)
        self._fusion = ffi.load_fusion()
        self._x = (ctypes.c_void_p * 4)(*[t.data_ptr() for t in (self.a, self.b, self.c, self.d)])
        self._g = (ctypes.c_void_p * 4)(*[t.data_ptr() for t in (self.da, self.db, self.dc, self.dd)])

    def _check(self, status):
        if status != 0:
            raise RuntimeError(self._fusion.mpChainError().decode())

    def forward(self):
        self._check(self._fusion.mpChainForward(self.expr, ffi.R32, self._x, self.e.data_ptr(), self.n, _ctx()))

    def reverse(self):
        self._check(self._fusion.mpChainReverse(self.expr, ffi.R32, self._x, self.de.data_ptr(), self._g, 0.0, self.n, _ctx()))


class _Vocab(Workload):
    dtype, has_reverse = torch.float32, True  # the configs name the forward; the reverse is measured beside it

    def __init__(self, seed=0, shape=None):
        self.shape = shape or self.shape
        m, n = self.shape
        g = _gen(seed)
        self.x = 3.0 * torch.randn(self.shape, generator=g, device="cuda", dtype=torch.float32)
        spike = torch.randint(0, n, (m,), generator=g, device="cuda")
        self.x[torch.arange(m, device="cuda"), spike] += 12.0
        self.y = torch.empty_like(self.x)
        self.dy = torch.randn(self.shape, generator=g, device="cuda", dtype=torch.float32)
        self.dx = torch.empty_like(self.x)
        self.scratch = softmax_scratch(torch.float32, m, n)
        self.rev_scratch = softmax_reverse_scratch(torch.float32, m, n)
        self.rows = m
        self.fwd_bytes = 2 * m * n * 4
        self.rev_bytes = 3 * m * n * 4

    def forward(self):
        softmax_forward(self.x, self.y, self.scratch)

    def reverse(self):
        softmax_reverse(self.y, self.dy, self.dx, 0.0, self.rev_scratch)


class Cfg5a(_Vocab):
    name = "cfg5a"
    shape = (512, 151936)


class Cfg5b(_Vocab):
    name = "cfg5b"
    shape = (2048, 50257)


class Copy(Workload):
    """Plain copy of known size (1 GiB in, 1 GiB out): the calibration run for the HBM traffic
    counters and the practical bandwidth ceiling next to which the other figures are read."""
    name, dtype, has_reverse = "copy", torch.float32, False
    n = 1 << 28

    def __init__(self, seed=0, n=None):
        self.n = n or self.n
        self.x = torch.randn((self.n,), generator=_gen(seed), device="cuda", dtype=torch.float32)
        self.y = torch.empty_like(self.x)
        self.rows = self.n
        self.fwd_bytes = 8 * self.n
        self.rev_bytes = 0

    def forward(self):
        _launch("copy", self.x.dtype, self.x.data_ptr(), self.y.data_ptr(), self.n)


class Permutate(Workload):
    name, dtype = "permutate", torch.float32
    shape = (16384, 16384)

    def __init__(self, seed=0, shape=None, dtype=None):
        self.shape = shape or self.shape
        self.dtype = dtype or self.dtype
        rows, cols = self.shape
        self.x = torch.randn(self.shape, generator=_gen(seed), device="cuda", dtype=torch.float32).to(self.dtype)
        self.y = torch.empty((cols, rows), dtype=self.dtype, device="cuda")
        self.gx = torch.zeros_like(self.x)
        self.rows = rows * cols
        self.fwd_bytes = 2 * self.x.numel() * self.x.element_size()
        self.rev_bytes = 3 * self.x.numel() * self.x.element_size()

    def forward(self):
        permutate(self.x, self.y)

    def reverse(self):  # src/ops/permutate.zig:58-69: the gradient comes back transposed and accumulates
        permutate(self.y, self.gx, 1.0)


class Gemm(Workload):
    name, dtype = "gemm", torch.float16
    mnk = (8192, 8192, 8192)

    def __init__(self, seed=0, mnk=None, dtype=None):
        self.mnk = mnk or self.mnk
        self.dtype = dtype or self.dtype
        m, n, k = self.mnk
        g = _gen(seed)
        self.a = (0.25 * torch.randn((m, n), generator=g, device="cuda")).to(self.dtype)
        self.b = (0.25 * torch.randn((n, k), generator=g, device="cuda")).to(self.dtype)
        self.gc = (0.25 * torch.randn((m, k), generator=g, device="cuda")).to(self.dtype)
        self.c = torch.empty((m, k), dtype=self.dtype, device="cuda")
        self.ga, self.gb = torch.zeros_like(self.a), torch.zeros_like(self.b)
        es = self.a.element_size()
        self.rows = m
        self.fwd_flops = 2 * m * n * k
        self.rev_flops = 4 * m * n * k
        self.fwd_bytes = (m * n + n * k + m * k) * es
        self.rev_bytes = (2 * m * k + 2 * n * k + 2 * m * n + m * n + n * k) * es

    def forward(self):
        m, n, k = self.mnk
        inner_product("ij_jk_ik", self.a, self.b, 1.0, self.c, 0.0, m, n, k)

    def reverse(self):  # src/ops/inner_product.zig:305-326 without the scratch transposes
        m, n, k = self.mnk
        inner_product("ij_kj_ik", self.gc, self.b, 1.0, self.ga, 1.0, m, k, n)
        inner_product("ji_jk_ik", self.a, self.gc, 1.0, self.gb, 1.0, n, m, k)


class NormVocab(Cfg2):
    """RMSNorm over rows as long as cfg5a's: every row shared by several workgroups, in both
    directions (no BASELINE configuration; here so that those kernels can be traced)."""
    name = "normvocab"
    shape = (512, 151936)

    def __init__(self, seed=0, shape=None):
        super().__init__(seed, shape)
        self.fwd_scratch = rmsnorm_scratch(torch.float32, *self.shape)

    def forward(self):
        rmsnorm_forward(self.x, self.gain, self.y, self.eps, self.fwd_scratch)


WORKLOADS = {c.name: c for c in (Cfg1, Cfg2, Cfg3, Cfg4, Cfg4Mid, Cfg5a, Cfg5b, Copy, Permutate, Gemm, RuntimeChain, NormVocab)}

DESCRIPTION = {
    "cfg1": "softmax fwd r32 [256,1024]",
    "cfg2": "RMSNorm fwd+rev r32 [8192,4096], gain [4096], eps 1e-6",
    "cfg3": "causal attention-score softmax fwd+rev r16 [524288,2048]",
    "cfg4": "fused selu((a+b)*(c+d)) fwd+rev r32 flat 2^28",
    "cfg4mid": "fused selu((a+b)*(c+d)) fwd+rev r32 flat 2^23: the forward keeps its inputs in the memory-side cache (not a BASELINE configuration)",
    "cfg5a": "vocabulary softmax fwd (+rev) r32 [512,151936]",
    "cfg5b": "vocabulary softmax fwd (+rev) r32 [2048,50257]",
    "chain": "relu((a-b)*(c+d)) fwd+rev r32 flat 2^28, an expression no build listed, compiled at run time",
    "normvocab": "RMSNorm fwd+rev r32 [512,151936]: rows shared by several workgroups (not a BASELINE configuration)",
    "copy": "plain copy r32 flat 2^28 (calibration)",
    "permutate": "transpose r32 [16384,16384], reverse = accumulating transpose",
    "gemm": "matrix product r16 (fp32 accumulate) 8192^3 on rocBLAS, reverse = its two gradient products",
}
