"""Helpers of the GPU parity tests: call the launchers through the C-ABI on torch-owned
device memory, guard every buffer with canaries, and compare against the fp64 oracle with
the tolerances stated for this path."""
import sys

import numpy as np
import torch

from metaphor_amd import ffi

KEY = {torch.float16: ffi.R16, torch.float32: ffi.R32, torch.float64: ffi.R64}
NP_OF = {torch.float16: np.float16, torch.float32: np.float32, torch.float64: np.float64}

# r32: 1e-5 relative (softmax outputs: 1e-6 absolute); r16: 2e-3 relative with a floor of one
# r16 subnormal ulp, softmax outputs included; r64 is held to 1e-12 relative. "Relative" is against
# max(|ref|, RMS of the reference row or tensor), which keeps cancellation-prone entries
# (dx of softmax, dg of RMSNorm) meaningful.
RTOL = {torch.float16: 2e-3, torch.float32: 1e-5, torch.float64: 1e-12}
FLOOR = {torch.float16: 2.0 ** -24, torch.float32: 0.0, torch.float64: 0.0}

GUARD = 64
_SENTINEL = 12345.0


def say(msg):
    """Name the case before each GPU step, so a lost box still tells which one it was."""
    print(f"[gpu-case] {msg}", flush=True)
    sys.stdout.flush()


def lib():
    kernels, utils = ffi.load()
    return kernels, utils


# ---------------------------------------------------------------- the test build of the row launchers
#
# The shipped library has no regime switch. lib/libmp_kernels_diag.so holds the softmax / RMSNorm
# launchers and their workspace-size functions compiled with -DMP_DIAGNOSTICS, plus
# mpSetRowRegime / mpSetClusterTuning. While an override is in force the wrappers below call into
# that library; otherwise they call the shipped one.

ROW_STEMS = ("softmax_ij_j", "softmax_ij_j_reverse", "rmsnorm_ij_j", "rmsnorm_ij_j_reverse")
ROW_SIZE_FNS = ("mpSoftmaxScratchBytes", "mpSoftmaxReverseScratchBytes", "mpRmsnormScratchBytes",
                "mpRmsnormReverseScratchBytes")
_diag = {"lib": None, "regime": 0, "tuned": False, "deep": 0, "own_words": 1, "keep_input": 2}


def diag_lib():
    if _diag["lib"] is None:
        import ctypes
        import os
        path = os.path.join(ffi.LIB_DIR, "libmp_kernels_diag.so")
        if not os.path.exists(path):
            raise ffi.BoundaryMissing(f"{path} is not built; run `python -m metaphor_amd.kernelgen`")
        ffi.load()  # the shipped library first: the test build must not shadow it
        d = ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)
        wanted = {f"launch_{s}_{t}" for s in ROW_STEMS for t in ("r16", "r32", "r64")} | set(ROW_SIZE_FNS)
        for ret, name, args in ffi.parse_declarations():
            if name in wanted:
                fn = getattr(d, name)
                fn.argtypes = [ffi._CTYPE[t] for t, _ in args]
                fn.restype = None if ret == "void" else ffi._CTYPE[ret]
        d.mpSetRowRegime.argtypes = [ffi.len_t]
        d.mpSetRowRegime.restype = None
        d.mpSetClusterTuning.argtypes = [ffi.len_t, ffi.len_t]
        d.mpSetClusterTuning.restype = None
        d.mpSetClusterDeep.argtypes = [ffi.len_t]
        d.mpSetClusterDeep.restype = None
        d.mpSetClusterWords.argtypes = [ffi.len_t]
        d.mpSetClusterWords.restype = None
        d.mpSetKeepInput.argtypes = [ffi.len_t]
        d.mpSetKeepInput.restype = None
        _diag["lib"] = d
    return _diag["lib"]


def _override_active():
    return _diag["regime"] != 0 or _diag["tuned"] or _diag["deep"] != 0 or _diag["own_words"] != 1 or _diag["keep_input"] != 2


def row_size(fn, dtype, m, n):
    """Workspace bytes from the library that will run the launch."""
    src = diag_lib() if _override_active() else lib()[0]
    return int(getattr(src, fn)(KEY[dtype], m, n))


def ctx():
    return ffi.StreamContext.from_handle(torch.cuda.current_stream().cuda_stream)


class Guarded:
    """A device tensor inside a larger buffer whose margins hold a sentinel. `shift`
    elements move the view off 16-byte alignment."""

    def __init__(self, shape, dtype, shift=0, fill=None):
        n = int(np.prod(shape)) if len(shape) else 1
        # keep the interior 16-byte aligned at shift 0: GUARD elements of any dtype are >= 128 bytes
        self.sentinel = _SENTINEL if dtype.is_floating_point else 165
        self.buf = torch.full((n + 2 * GUARD + shift,), self.sentinel, dtype=dtype, device="cuda")
        self.lo = GUARD + shift
        self.t = self.buf[self.lo:self.lo + n].view(*shape) if n else self.buf[self.lo:self.lo].view(*shape)
        if fill is not None:
            self.t.copy_(fill)

    def check(self, what):
        lo = self.buf[:self.lo]
        hi = self.buf[self.lo + self.t.numel():]
        ok = bool((lo == self.sentinel).all()) and bool((hi == self.sentinel).all())
        assert ok, f"{what}: wrote outside its buffer"


def dev(a, dtype, shift=0):
    """numpy -> guarded device tensor of `dtype` (values rounded to the storage type first)."""
    t = torch.from_numpy(np.ascontiguousarray(a)).to(dtype)
    g = Guarded(tuple(t.shape), dtype, shift)
    g.t.copy_(t)
    return g


def host(t):
    """device tensor -> numpy in its storage dtype (what the oracle must read)."""
    return t.detach().cpu().numpy()


def parity_stats(got, ref, dtype, rowwise=True, rtol=None, atol=None, scale=None):
    """Numbers of one comparison, without judging it: the error of `got` against the fp64
    reference and the bound  rtol * max(|ref|, RMS(ref row|tensor), scale) + floor  (or a plain
    atol). Returns a dict: n, max_abs (largest |got - ref|), max_rel (largest error over
    max(|ref|, RMS), the form the tolerance is stated in), worst (largest error over its bound:
    below 1 means inside), violations, and where the worst entry is."""
    g = got.detach().double().cpu().numpy()
    ref = np.asarray(ref, dtype=np.float64)
    assert g.shape == ref.shape, f"shape {g.shape} vs {ref.shape}"
    if g.size == 0:
        return {"n": 0, "max_abs": 0.0, "max_rel": 0.0, "worst": 0.0, "violations": 0, "at": None}
    both_nan = np.isnan(g) & np.isnan(ref)
    fin = np.where(np.isfinite(ref), ref, 0.0)
    if rowwise and ref.ndim >= 2:
        rms = np.sqrt((fin ** 2).mean(axis=-1, keepdims=True))
    else:
        rms = np.sqrt((fin ** 2).mean())
    plain = np.maximum(np.abs(fin), rms)
    if atol is not None:
        bound = np.full_like(ref, atol)
    else:
        rtol = RTOL[dtype] if rtol is None else rtol
        mag = plain if scale is None else np.maximum(plain, np.asarray(scale, dtype=np.float64))
        bound = rtol * mag + FLOOR[dtype]
    with np.errstate(invalid="ignore", divide="ignore"):
        err = np.where(both_nan | ((g == ref) & ~np.isnan(ref)), 0.0, np.abs(g - ref))
        bad = ~(err <= bound)
        ratio = np.where(bad & ~np.isfinite(err), np.inf, err / np.maximum(bound, 1e-300))
        rel = np.where(np.isfinite(err), err / np.maximum(plain, 1e-300), np.inf)
    at = np.unravel_index(np.argmax(ratio), ref.shape)
    finite_err = np.where(np.isfinite(err), err, 0.0)
    return {"n": int(ref.size), "max_abs": float(finite_err.max()), "max_rel": float(np.where(plain > 0, rel, 0.0).max()),
            "worst": float(ratio[at]), "violations": int(bad.sum()), "at": tuple(int(i) for i in at),
            "got": float(g[at]), "ref": float(ref[at]), "err": float(err[at]), "bound": float(bound[at])}


PARITY_LOG = []  # (what, stats) of every comparison of this process, in order


def compare(got, ref, dtype, what, rowwise=True, rtol=None, atol=None, scale=None):
    """|got - ref| <= rtol * max(|ref|, RMS(ref row|tensor), scale) + floor (or a plain atol).

    `scale` is the magnitude of the terms an entry is the difference of (see
    softmax_reverse_scale / rmsnorm_reverse_scales): where two terms of size s cancel to a
    result far below s, no fp32 kernel can be closer than a few ulp of s. Prints and returns
    the numbers of the comparison (parity_stats); raises when an entry is outside its bound."""
    st = parity_stats(got, ref, dtype, rowwise, rtol, atol, scale)
    PARITY_LOG.append((what, st))
    if st["n"]:
        plain = ""
        if scale is not None:  # how the same result stands against the bound without the scale term
            p = parity_stats(got, ref, dtype, rowwise, rtol, atol, None)
            plain = f" (without scale: worst {p['worst']:.3f}, violations {p['violations']})"
        print(f"[parity] {what}: n={st['n']} max_abs={st['max_abs']:.3e} max_rel={st['max_rel']:.3e} "
              f"worst err/bound={st['worst']:.3f} violations={st['violations']}{plain}", flush=True)
    if st["violations"]:
        raise AssertionError(
            f"{what}: {st['violations']} of {st['n']} outside tolerance; worst at {st['at']}: "
            f"got {st['got']!r} ref {st['ref']!r} err {st['err']:.3e} bound {st['bound']:.3e}")
    return st


def softmax_tol(dtype):
    """Keyword arguments of compare() for softmax outputs: r32 within 1e-6 absolute (r64 1e-13);
    r16 like every other r16 result, 2e-3 * max(|ref|, RMS of the row) + one r16 subnormal ulp."""
    return {} if dtype == torch.float16 else {"atol": 1e-6 if dtype == torch.float32 else 1e-13}


def softmax_reverse_scale(y, dy, dx_in=None, alpha=0.0):
    """dx = y*dy - y*dot (+ alpha*old): size of the terms that cancel."""
    y, dy = np.asarray(y, np.float64), np.asarray(dy, np.float64)
    s = np.abs(y) * (np.abs(dy) + np.abs(y * dy).sum(axis=-1, keepdims=True))
    if dx_in is not None:
        s = s + abs(alpha) * np.abs(np.asarray(dx_in, np.float64))
    return s


def rmsnorm_reverse_scales(x, g, dy, eps, dx_in=None, dg_in=None, alpha=0.0):
    """dx = r*dy*g - r^3*x*c: the size of its two terms (they cancel completely for rows of one
    element, and largely for rows of a few). The second value, for dg = sum_i dy*x*r, is None: the
    gain gradient is held to the plain bound rtol * max(|ref|, RMS(ref)). Over the 2064 dg
    comparisons of this suite its worst error is 0.24 of that bound (16-row fp32 partial sums and an
    fp64 finish leave no visible cancellation error)."""
    x, g, dy = (np.asarray(a, np.float64) for a in (x, g, dy))
    n = x.shape[-1]
    r = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
    c_abs = np.abs(dy * g * x).sum(axis=-1, keepdims=True) / n
    sdx = r * (np.abs(dy * g) + np.abs(x) * r * r * c_abs)
    if dx_in is not None:
        sdx = sdx + abs(alpha) * np.abs(np.asarray(dx_in, np.float64))
    return sdx, None


# ---------------------------------------------------------------- launcher wrappers

def _call(stem, dtype, *args):
    if stem in ROW_STEMS and _override_active():
        name = f"launch_{stem}_" + ("r16", "r32", "r64")[KEY[dtype]]
        getattr(diag_lib(), name)(*args, ctx())
        return
    kernels, _ = lib()
    ffi.invoke(getattr(kernels, stem), KEY[dtype], *args, ctx())


def addition(a, b, c):
    _call("addition", a.dtype, a.data_ptr(), b.data_ptr(), c.data_ptr(), a.numel())


def hadamard(a, b, c):
    _call("hadamard", a.dtype, a.data_ptr(), b.data_ptr(), c.data_ptr(), a.numel())


def hadamard_reverse(a, b, c):
    _call("hadamard_reverse", a.dtype, a.data_ptr(), b.data_ptr(), c.data_ptr(), a.numel())


def subtraction(a, b, c):
    _call("subtraction", a.dtype, a.data_ptr(), b.data_ptr(), c.data_ptr(), a.numel())


def unary(stem, a, b):
    """negate, relu, stepwise, copy, selu: (src, dst, n)."""
    _call(stem, a.dtype, a.data_ptr(), b.data_ptr(), a.numel())


def relu_reverse(a_value, a_grads, b_grads):
    _call("relu_reverse", a_value.dtype, a_value.data_ptr(), a_grads.data_ptr(), b_grads.data_ptr(),
          a_value.numel())


def scalar_op(stem, a, value, c):
    """dilate, dilate_reverse, translate: (a, value, c, n)."""
    _call(stem, a.dtype, a.data_ptr(), float(value), c.data_ptr(), a.numel())


def fill(a, value):
    _call("fill", a.dtype, a.data_ptr(), float(value), a.numel())


def sequence(a, init, step):
    _call("sequence", a.dtype, a.data_ptr(), float(init), float(step), a.numel())


def selu(a, b):
    _call("selu", a.dtype, a.data_ptr(), b.data_ptr(), a.numel())


def selu_reverse(a_value, a_grads, b_grads):
    _call("selu_reverse", a_value.dtype, a_value.data_ptr(), a_grads.data_ptr(), b_grads.data_ptr(),
          a_value.numel())


def fused(a, b, c, d, e):
    _call("fused_selu_hadamard_add_add", a.dtype, a.data_ptr(), b.data_ptr(), c.data_ptr(),
          d.data_ptr(), e.data_ptr(), a.numel())


def fused_reverse(a, b, c, d, de, da, db, dc, dd, alpha=0.0):
    _call("fused_selu_hadamard_add_add_reverse", a.dtype, a.data_ptr(), b.data_ptr(), c.data_ptr(),
          d.data_ptr(), de.data_ptr(), da.data_ptr(), db.data_ptr(), dc.data_ptr(), dd.data_ptr(),
          float(alpha), a.numel())


def _pointer_array(tensors):
    import ctypes
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def chain_forward(expr, xs, out):
    """An expression fused at run time: returns the entry point's status (0 = enqueued)."""
    f = ffi.load_fusion()
    return f.mpChainForward(expr.encode(), KEY[out.dtype], _pointer_array(xs), out.data_ptr(), out.numel(), ctx())


def chain_reverse(expr, xs, out_grads, grads, alpha=0.0):
    f = ffi.load_fusion()
    return f.mpChainReverse(expr.encode(), KEY[out_grads.dtype], _pointer_array(xs), out_grads.data_ptr(),
                            _pointer_array(grads), float(alpha), out_grads.numel(), ctx())


def chain_forward_many(exprs, xs, outs):
    """Several results over the same leaves ("e1;e2") in one kernel."""
    f = ffi.load_fusion()
    return f.mpChainForwardMany(exprs.encode(), KEY[outs[0].dtype], _pointer_array(xs), _pointer_array(outs),
                                outs[0].numel(), ctx())


def chain_reverse_many(exprs, xs, out_grads, grads, alpha=0.0):
    f = ffi.load_fusion()
    return f.mpChainReverseMany(exprs.encode(), KEY[grads[0].dtype], _pointer_array(xs), _pointer_array(out_grads),
                                _pointer_array(grads), float(alpha), grads[0].numel(), ctx())


def chain_error():
    return ffi.load_fusion().mpChainError().decode()


def matrix_op(stem, src, dst, alpha, m, n):
    """reduce_ij_i, reduce_ij_j, broadcast_i_ij, broadcast_j_ij: (src, dst, alpha, m, n)."""
    _call(stem, src.dtype, src.data_ptr(), dst.data_ptr(), float(alpha), m, n)


def reduce_ij_j_scratch(src, dst, alpha, m, n, scratch="auto"):
    """Column sums through the workspace-taking launcher; "auto" sizes the workspace, None passes NULL."""
    guard = None
    if isinstance(scratch, str):
        kernels, _ = lib()
        nbytes = int(kernels.mpReduceScratchBytes(KEY[src.dtype], m, n))
        guard = Guarded((nbytes,), torch.uint8) if nbytes else None
        scratch = guard.t if guard is not None else None
    _call("reduce_ij_j_scratch", src.dtype, src.data_ptr(), dst.data_ptr(),
          scratch.data_ptr() if scratch is not None else None, float(alpha), m, n)
    if guard is not None:
        torch.cuda.synchronize()
        guard.check("reduce scratch")
    return guard is not None


def softmax_scratch(dtype, m, n):
    nbytes = row_size("mpSoftmaxScratchBytes", dtype, m, n)
    return (Guarded((nbytes,), torch.uint8) if nbytes else None), nbytes


def softmax(x, y, scratch="auto"):
    """scratch: "auto" sizes and passes the workspace the launcher asks for, None passes NULL."""
    m, n = x.shape
    guard = None
    if isinstance(scratch, str):
        guard, _ = softmax_scratch(x.dtype, m, n)
        scratch = guard.t if guard is not None else None
    _call("softmax_ij_j", x.dtype, x.data_ptr(), y.data_ptr(),
          scratch.data_ptr() if scratch is not None else None, m, n)
    if guard is not None:
        torch.cuda.synchronize()
        guard.check("softmax scratch")


def softmax_reverse(y, dy, dx, alpha=0.0, scratch="auto"):
    """scratch: "auto" sizes and passes the workspace the launcher asks for, None passes NULL."""
    m, n = y.shape
    guard = None
    if isinstance(scratch, str):
        nbytes = row_size("mpSoftmaxReverseScratchBytes", y.dtype, m, n)
        guard = Guarded((nbytes,), torch.uint8) if nbytes else None
        scratch = guard.t if guard is not None else None
    _call("softmax_ij_j_reverse", y.dtype, y.data_ptr(), dy.data_ptr(), dx.data_ptr(),
          scratch.data_ptr() if scratch is not None else None, float(alpha), m, n)
    if guard is not None:
        torch.cuda.synchronize()
        guard.check("softmax reverse scratch")


def rmsnorm(x, g, y, eps, scratch="auto"):
    """scratch: "auto" sizes and passes the workspace the launcher asks for, None passes NULL."""
    m, n = x.shape
    guard = None
    if isinstance(scratch, str):
        nbytes = row_size("mpRmsnormScratchBytes", x.dtype, m, n)
        guard = Guarded((nbytes,), torch.uint8) if nbytes else None
        scratch = guard.t if guard is not None else None
    _call("rmsnorm_ij_j", x.dtype, x.data_ptr(), g.data_ptr(), y.data_ptr(),
          scratch.data_ptr() if scratch is not None else None, float(eps), m, n)
    if guard is not None:
        torch.cuda.synchronize()
        guard.check("rmsnorm scratch")


def rmsnorm_scratch(dtype, m, n):
    nbytes = row_size("mpRmsnormReverseScratchBytes", dtype, m, n)
    return Guarded((max(nbytes, 1),), torch.uint8), nbytes


def rmsnorm_reverse(x, g, dy, dx, dg, scratch, eps, alpha=0.0):
    m, n = x.shape
    _call("rmsnorm_ij_j_reverse", x.dtype, x.data_ptr(), g.data_ptr(), dy.data_ptr(), dx.data_ptr(),
          dg.data_ptr(), scratch.data_ptr(), float(eps), float(alpha), m, n)


def set_regime(r):
    """Force a row regime (0 = automatic) in the test build, which then serves the row launchers."""
    diag_lib().mpSetRowRegime(int(r))
    _diag["regime"] = int(r)


def set_cluster_tuning(packs_per_block=0, spin_limit=1 << 22):
    """Chunk size and poll limit of the shared-row kernels in the test build (defaults restore it)."""
    diag_lib().mpSetClusterTuning(int(packs_per_block), int(spin_limit))
    _diag["tuned"] = not (int(packs_per_block) == 0 and int(spin_limit) == 1 << 22)


def set_cluster_deep(which=0):
    """Which kernel the RMSNorm reverse runs on shared r32 rows in the test build: 0 by the launcher's
    rule, 1 always the pipelined one, 2 never."""
    diag_lib().mpSetClusterDeep(int(which))
    _diag["deep"] = int(which)


def set_cluster_words(own=1):
    """Where the shared-row softmax kernels of the test build keep their exchange words: 1 in the
    library's own memory (as shipped), 0 in the caller's workspace, cleared before every launch."""
    diag_lib().mpSetClusterWords(int(own))
    _diag["own_words"] = int(own)


def set_keep_input(mode=2):
    """How the resident RMSNorm forward of the test build loads x: 0 streaming loads, 1 loads that
    leave x in the memory-side cache, 2 by the size of the tensor (as shipped)."""
    diag_lib().mpSetKeepInput(int(mode))
    _diag["keep_input"] = int(mode)


def permutate(src, dst, alpha=0.0):
    rows, cols = src.shape
    _call("permutate_ij_ji", src.dtype, src.data_ptr(), dst.data_ptr(), float(alpha), rows, cols)


class BlasStream:
    """A stream context from mpInitStream: the only kind that carries the BLAS handle the
    matrix-product launchers need. Work on it is fenced against torch's stream by full
    device synchronisation on entry and a stream synchronisation after each call."""

    def __enter__(self):
        _, utils = lib()
        torch.cuda.synchronize()
        self.sc = utils.mpInitStream()
        assert self.sc.blas_handle.ptr
        return self

    def __exit__(self, *exc):
        _, utils = lib()
        utils.mpStreamSynchronize(self.sc)
        utils.mpDeinitStream(self.sc)

    def enqueue(self, stem, dtype, *args):
        """Any launcher on this stream, without waiting for it (sync() does)."""
        kernels, _ = lib()
        ffi.invoke(getattr(kernels, stem), KEY[dtype], *args, self.sc)

    def sync(self):
        _, utils = lib()
        utils.mpStreamSynchronize(self.sc)

    def matrix_op(self, stem, src, dst, alpha, m, n):
        """reduce_ij_j and its like on this stream, whose context owns a workspace."""
        kernels, utils = lib()
        torch.cuda.synchronize()
        getattr(kernels, stem)[KEY[src.dtype]](src.data_ptr(), dst.data_ptr(), float(alpha), m, n, self.sc)
        utils.mpStreamSynchronize(self.sc)

    def inner_product(self, form, a, b, alpha, c, beta, m, n, k):
        """form: "ij_jk_ik", "ij_kj_ik" or "ji_jk_ik"."""
        kernels, utils = lib()
        torch.cuda.synchronize()
        getattr(kernels, "inner_product_" + form)[KEY[a.dtype]](
            a.data_ptr(), b.data_ptr(), float(alpha), c.data_ptr(), float(beta), m, n, k, self.sc)
        utils.mpStreamSynchronize(self.sc)
