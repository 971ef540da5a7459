"""ctypes front end of the CPU oracle (oracle/libmp_oracle.so) for tests, smoke and the
benchmark's cpu_baseline leg. Inputs are numpy arrays of float16/float32/float64; every
result comes back as float64, unrounded."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")
_SO = os.path.join(_ORACLE_DIR, "libmp_oracle.so")

_KEY = {np.dtype(np.float16): 0, np.dtype(np.float32): 1, np.dtype(np.float64): 2}


def _load():
    if not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _ORACLE_DIR, "-s"])
    return ctypes.CDLL(_SO)


_lib = _load()
_lib.oracle_threads.restype = ctypes.c_int
_lib.oracle_double_to_half_bits.restype = ctypes.c_uint16
_lib.oracle_double_to_half_bits.argtypes = [ctypes.c_double]
_lib.oracle_half_bits_to_double.restype = ctypes.c_double
_lib.oracle_half_bits_to_double.argtypes = [ctypes.c_uint16]

_vp = ctypes.c_void_p
_sz = ctypes.c_size_t
_db = ctypes.c_double
_it = ctypes.c_int


def _sig(name, *argtypes):
    fn = getattr(_lib, name)
    fn.argtypes = list(argtypes)
    fn.restype = None
    return fn


_addition = _sig("oracle_addition", _it, _vp, _vp, _vp, _sz)
_hadamard = _sig("oracle_hadamard", _it, _vp, _vp, _vp, _sz)
_hadamard_reverse = _sig("oracle_hadamard_reverse", _it, _vp, _vp, _vp, _vp, _sz)
_selu = _sig("oracle_selu", _it, _vp, _vp, _sz)
_selu_reverse = _sig("oracle_selu_reverse", _it, _vp, _vp, _vp, _vp, _sz)
_fused = _sig("oracle_fused_selu_hadamard_add_add", _it, _vp, _vp, _vp, _vp, _vp, _sz)
_fused_rev = _sig("oracle_fused_selu_hadamard_add_add_reverse", _it, *([_vp] * 13), _db, _sz)
_reduce_i = _sig("oracle_reduce_ij_i", _it, _vp, _vp, _vp, _db, _sz, _sz)
_reduce_j = _sig("oracle_reduce_ij_j", _it, _vp, _vp, _vp, _db, _sz, _sz)
_bcast_i = _sig("oracle_broadcast_i_ij", _it, _vp, _vp, _vp, _db, _sz, _sz)
_bcast_j = _sig("oracle_broadcast_j_ij", _it, _vp, _vp, _vp, _db, _sz, _sz)
_softmax = _sig("oracle_softmax_ij_j", _it, _vp, _vp, _sz, _sz)
_softmax_rev = _sig("oracle_softmax_ij_j_reverse", _it, _vp, _vp, _vp, _vp, _db, _sz, _sz)
_rmsnorm = _sig("oracle_rmsnorm_ij_j", _it, _vp, _vp, _vp, _db, _sz, _sz)
_rmsnorm_rev = _sig("oracle_rmsnorm_ij_j_reverse", _it, *([_vp] * 7), _db, _db, _sz, _sz)
_rmsnorm_rev_mt = _sig("oracle_rmsnorm_ij_j_reverse_mt", _it, *([_vp] * 5), _db, _sz, _sz)
_set_threads = _sig("oracle_set_threads", _it)
_subtraction = _sig("oracle_subtraction", _it, _vp, _vp, _vp, _sz)
_negate = _sig("oracle_negate", _it, _vp, _vp, _sz)
_relu = _sig("oracle_relu", _it, _vp, _vp, _sz)
_relu_reverse = _sig("oracle_relu_reverse", _it, _vp, _vp, _vp, _vp, _sz)
_stepwise = _sig("oracle_stepwise", _it, _vp, _vp, _sz)
_dilate = _sig("oracle_dilate", _it, _vp, _db, _vp, _sz)
_dilate_reverse = _sig("oracle_dilate_reverse", _it, _vp, _db, _vp, _vp, _sz)
_translate = _sig("oracle_translate", _it, _vp, _db, _vp, _sz)
_fill = _sig("oracle_fill", _it, _db, _vp, _sz)
_sequence = _sig("oracle_sequence", _it, _db, _db, _vp, _sz)
_copy = _sig("oracle_copy", _it, _vp, _vp, _sz)
_permutate = _sig("oracle_permutate_ij_ji", _it, _vp, _vp, _vp, _db, _sz, _sz)
_inner = _sig("oracle_inner_product", _it, _it, _it, _vp, _vp, _db, _vp, _db, _vp, _vp, _sz, _sz, _sz)


def threads():
    return int(_lib.oracle_threads())


def set_threads(t):
    _set_threads(int(t))


def _prep(*arrays):
    """Contiguous copies sharing one dtype; returns (key, arrays)."""
    first = next(a for a in arrays if a is not None)
    dt = np.dtype(first.dtype)
    if dt not in _KEY:
        raise TypeError(f"unsupported dtype {dt}")
    out = []
    for a in arrays:
        if a is None:
            out.append(None)
            continue
        if a.dtype != dt:
            raise TypeError("all operands must share one dtype")
        out.append(np.ascontiguousarray(a))
    return _KEY[dt], out


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _out(shape):
    return np.empty(shape, dtype=np.float64)


def addition(a, b):
    k, (a, b) = _prep(a, b)
    c = _out(a.shape)
    _addition(k, _p(a), _p(b), _p(c), a.size)
    return c


def hadamard(a, b):
    k, (a, b) = _prep(a, b)
    c = _out(a.shape)
    _hadamard(k, _p(a), _p(b), _p(c), a.size)
    return c


def hadamard_reverse(a, b, c_in=None):
    k, (a, b, c_in) = _prep(a, b, c_in)
    c = _out(a.shape)
    _hadamard_reverse(k, _p(a), _p(b), _p(c_in), _p(c), a.size)
    return c


def subtraction(a, b):
    k, (a, b) = _prep(a, b)
    c = _out(a.shape)
    _subtraction(k, _p(a), _p(b), _p(c), a.size)
    return c


def _unary(fn, a):
    k, (a,) = _prep(a)
    b = _out(a.shape)
    fn(k, _p(a), _p(b), a.size)
    return b


def negate(a):
    return _unary(_negate, a)


def relu(a):
    return _unary(_relu, a)


def stepwise(a):
    return _unary(_stepwise, a)


def copy(a):
    return _unary(_copy, a)


def relu_reverse(a_value, b_grads, a_grads_in=None):
    k, (a_value, b_grads, a_grads_in) = _prep(a_value, b_grads, a_grads_in)
    o = _out(a_value.shape)
    _relu_reverse(k, _p(a_value), _p(a_grads_in), _p(b_grads), _p(o), a_value.size)
    return o


def dilate(a, value):
    k, (a,) = _prep(a)
    c = _out(a.shape)
    _dilate(k, _p(a), float(value), _p(c), a.size)
    return c


def dilate_reverse(a, value, b_in=None):
    k, (a, b_in) = _prep(a, b_in)
    b = _out(a.shape)
    _dilate_reverse(k, _p(a), float(value), _p(b_in), _p(b), a.size)
    return b


def translate(a, value):
    k, (a,) = _prep(a)
    c = _out(a.shape)
    _translate(k, _p(a), float(value), _p(c), a.size)
    return c


def fill(dtype, value, n):
    a = _out((n,))
    _fill(_KEY[np.dtype(dtype)], float(value), _p(a), n)
    return a


def sequence(dtype, init, step, n):
    a = _out((n,))
    _sequence(_KEY[np.dtype(dtype)], float(init), float(step), _p(a), n)
    return a


def selu(a):
    k, (a,) = _prep(a)
    b = _out(a.shape)
    _selu(k, _p(a), _p(b), a.size)
    return b


def selu_reverse(a_value, b_grads, a_grads_in=None):
    k, (a_value, b_grads, a_grads_in) = _prep(a_value, b_grads, a_grads_in)
    o = _out(a_value.shape)
    _selu_reverse(k, _p(a_value), _p(a_grads_in), _p(b_grads), _p(o), a_value.size)
    return o


def fused_selu_hadamard_add_add(a, b, c, d):
    k, (a, b, c, d) = _prep(a, b, c, d)
    e = _out(a.shape)
    _fused(k, _p(a), _p(b), _p(c), _p(d), _p(e), a.size)
    return e


def fused_selu_hadamard_add_add_reverse(a, b, c, d, de, grads_in=None, alpha=0.0):
    gi = grads_in if grads_in is not None else (None, None, None, None)
    k, arrs = _prep(a, b, c, d, de, *gi)
    a, b, c, d, de = arrs[:5]
    gi = arrs[5:]
    outs = [_out(a.shape) for _ in range(4)]
    _fused_rev(k, _p(a), _p(b), _p(c), _p(d), _p(de), *[_p(g) for g in gi],
               *[_p(o) for o in outs], float(alpha), a.size)
    return tuple(outs)


def reduce_ij_i(src, dst_in=None, alpha=0.0):
    k, (src, dst_in) = _prep(src, dst_in)
    m, n = src.shape
    dst = _out((m,))
    _reduce_i(k, _p(src), _p(dst_in), _p(dst), float(alpha), m, n)
    return dst


def reduce_ij_j(src, dst_in=None, alpha=0.0):
    k, (src, dst_in) = _prep(src, dst_in)
    m, n = src.shape
    dst = _out((n,))
    _reduce_j(k, _p(src), _p(dst_in), _p(dst), float(alpha), m, n)
    return dst


def broadcast_i_ij(src, m, n, dst_in=None, alpha=0.0):
    k, (src, dst_in) = _prep(src, dst_in)
    dst = _out((m, n))
    _bcast_i(k, _p(src), _p(dst_in), _p(dst), float(alpha), m, n)
    return dst


def broadcast_j_ij(src, m, n, dst_in=None, alpha=0.0):
    k, (src, dst_in) = _prep(src, dst_in)
    dst = _out((m, n))
    _bcast_j(k, _p(src), _p(dst_in), _p(dst), float(alpha), m, n)
    return dst


def permutate_ij_ji(src, dst_in=None, alpha=0.0):
    k, (src, dst_in) = _prep(src, dst_in)
    rows, cols = src.shape
    dst = _out((cols, rows))
    _permutate(k, _p(src), _p(dst_in), _p(dst), float(alpha), rows, cols)
    return dst


def inner_product(a, b, alpha=1.0, c_in=None, beta=0.0, ta=False, tb=False, with_scale=False):
    """c[m,k] = alpha * op(a) . op(b) + beta * c_in; a is stored [n,m] when ta, b [k,n] when tb."""
    key, (a, b, c_in) = _prep(a, b, c_in)
    m, n = (a.shape[1], a.shape[0]) if ta else a.shape
    k = b.shape[0] if tb else b.shape[1]
    assert (b.shape[1] if tb else b.shape[0]) == n
    c = _out((m, k))
    scale = _out((m, k))
    _inner(key, int(ta), int(tb), _p(a), _p(b), float(alpha), _p(c_in), float(beta), _p(c), _p(scale), m, n, k)
    return (c, scale) if with_scale else c


def softmax_ij_j(x):
    k, (x,) = _prep(x)
    m, n = x.shape
    y = _out(x.shape)
    _softmax(k, _p(x), _p(y), m, n)
    return y


def softmax_ij_j_reverse(y, dy, dx_in=None, alpha=0.0):
    k, (y, dy, dx_in) = _prep(y, dy, dx_in)
    m, n = y.shape
    dx = _out(y.shape)
    _softmax_rev(k, _p(y), _p(dy), _p(dx_in), _p(dx), float(alpha), m, n)
    return dx


def rmsnorm_ij_j(x, g, eps):
    k, (x, g) = _prep(x, g)
    m, n = x.shape
    y = _out(x.shape)
    _rmsnorm(k, _p(x), _p(g), _p(y), float(eps), m, n)
    return y


def rmsnorm_ij_j_reverse(x, g, dy, eps, dx_in=None, dg_in=None, alpha=0.0):
    k, (x, g, dy, dx_in, dg_in) = _prep(x, g, dy, dx_in, dg_in)
    m, n = x.shape
    dx, dg = _out(x.shape), _out((n,))
    _rmsnorm_rev(k, _p(x), _p(g), _p(dy), _p(dx_in), _p(dg_in), _p(dx), _p(dg),
                 float(eps), float(alpha), m, n)
    return dx, dg


def rmsnorm_ij_j_reverse_mt(x, g, dy, eps):
    """Row-parallel form used only for timing the CPU baseline."""
    k, (x, g, dy) = _prep(x, g, dy)
    m, n = x.shape
    dx, dg = _out(x.shape), _out((n,))
    _rmsnorm_rev_mt(k, _p(x), _p(g), _p(dy), _p(dx), _p(dg), float(eps), m, n)
    return dx, dg


def double_to_half_bits(x):
    return int(_lib.oracle_double_to_half_bits(float(x)))


def half_bits_to_double(h):
    return float(_lib.oracle_half_bits_to_double(int(h)))
