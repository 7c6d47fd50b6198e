"""ctypes front end of the CPU checker in ``fft_oracle.c``.

TEST INFRASTRUCTURE ONLY: imported by the test-suite, the smoke check and the
benchmark's CPU-baseline leg; the shipped library never touches it.

The C side is compiled twice (double ``_d`` and long double ``_ld``
arithmetic); ``ld=True`` selects the long double build, used as the reference
for fp64 parity.  All arrays cross the boundary as float64.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

COMPLEX_FORWARD, COMPLEX_INVERSE, REAL_FORWARD, REAL_INVERSE = 0, 1, 2, 3


def build(force=False):
    """Compile liborc.so with gcc (no GPU code involved)."""
    so = os.path.join(_HERE, "liborc.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-s", "-C", _HERE, "clean"])
        subprocess.check_call(["make", "-s", "-C", _HERE])
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liborc.so")
        if not os.path.exists(so):
            build()
        _LIB = ctypes.CDLL(so)
    return _LIB


def _fn(name, ld):
    return getattr(lib(), name + ("_ld" if ld else "_d"))


def _dptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def _as_ri(x):
    """complex array -> contiguous float64 (re, im) pairs (copy)."""
    x = np.ascontiguousarray(x, dtype=np.complex128)
    return x.view(np.float64).copy()


def dft_naive(x, direction=-1, ld=True):
    """O(n^2) DFT by definition of a 1D complex array."""
    a = _as_ri(x)
    out = np.empty_like(a)
    _fn("orc_dft_naive", ld)(_dptr(a), _dptr(out), ctypes.c_size_t(x.size), ctypes.c_int(direction))
    return out.view(np.complex128)


def dft_bin(x, k, direction=-1, ld=True):
    a = _as_ri(x)
    out = np.empty(2, dtype=np.float64)
    _fn("orc_dft_bin", ld)(_dptr(a), ctypes.c_size_t(x.size), ctypes.c_size_t(k),
                           ctypes.c_int(direction), _dptr(out))
    return complex(out[0], out[1])


def factorize(n):
    f = (ctypes.c_int * 64)()
    nf = lib().orc_factorize_d(ctypes.c_size_t(n), f, ctypes.c_int(64))
    return [int(f[i]) for i in range(max(nf, 0))]


def stacked_twiddles(n, factors, ld=True):
    f = (ctypes.c_int * len(factors))(*factors)
    fn = _fn("orc_stacked_twiddles", ld)
    fn.restype = ctypes.c_size_t
    cnt = fn(ctypes.c_size_t(n), f, ctypes.c_int(len(factors)), None)
    out = np.empty(2 * cnt, dtype=np.float64)
    fn(ctypes.c_size_t(n), f, ctypes.c_int(len(factors)), _dptr(out))
    return out.view(np.complex128)


def stockham(x, factors, direction=-1, ld=True):
    a = _as_ri(x)
    f = (ctypes.c_int * len(factors))(*factors)
    _fn("orc_stockham", ld)(_dptr(a), ctypes.c_size_t(x.size), f, ctypes.c_int(len(factors)),
                            ctypes.c_int(direction))
    return a.view(np.complex128)


def fft1d(x, direction=-1, ld=False):
    """Batched contiguous 1D complex transform along the last axis."""
    x = np.asarray(x)
    n = x.shape[-1]
    batch = x.size // n
    a = _as_ri(x)
    _fn("orc_fft1d", ld)(_dptr(a), ctypes.c_size_t(n), ctypes.c_size_t(batch), ctypes.c_int(direction))
    return a.view(np.complex128).reshape(x.shape)


def bluestein1d(x, direction=-1, ld=True):
    a = _as_ri(x)
    _fn("orc_bluestein1d", ld)(_dptr(a), ctypes.c_size_t(x.size), ctypes.c_int(direction))
    return a.view(np.complex128)


def large_twiddle(L, base, steps, u, ld=True):
    out = np.empty(2, dtype=np.float64)
    _fn("orc_large_twiddle", ld)(ctypes.c_size_t(L), ctypes.c_int(base), ctypes.c_int(steps),
                                 ctypes.c_uint64(u), _dptr(out))
    return complex(out[0], out[1])


def large1d_cc(x, n1, n0, base, steps, direction=-1, ld=True):
    a = _as_ri(x)
    assert x.size == n1 * n0
    _fn("orc_large1d_cc", ld)(_dptr(a), ctypes.c_size_t(n1), ctypes.c_size_t(n0), ctypes.c_int(base),
                              ctypes.c_int(steps), ctypes.c_int(direction))
    return a.view(np.complex128)


def r2c_post(z, ld=True):
    half = z.size
    a = _as_ri(z)
    out = np.empty(2 * (half + 1), dtype=np.float64)
    _fn("orc_r2c_post", ld)(_dptr(a), _dptr(out), ctypes.c_size_t(half))
    return out.view(np.complex128)


def c2r_pre(h, ld=True):
    half = h.size - 1
    a = _as_ri(h)
    out = np.empty(2 * half, dtype=np.float64)
    _fn("orc_c2r_pre", ld)(_dptr(a), _dptr(out), ctypes.c_size_t(half))
    return out.view(np.complex128)


def transform(kind, lengths, batch, x, ld=False):
    """Whole transform at the API's default contiguous layout.

    ``lengths[0]`` is the fastest-varying dimension (rocfft.h convention), so a
    numpy array for lengths (n0, n1, n2) has shape (batch, n2, n1, n0).
    Returns a flat array: complex128 (kinds 0, 1, 2) or float64 (kind 3).
    """
    lengths = [int(v) for v in lengths]
    total = int(np.prod(lengths))
    h0 = lengths[0] // 2 + 1
    htotal = total // lengths[0] * h0
    if kind in (COMPLEX_FORWARD, COMPLEX_INVERSE):
        a = _as_ri(np.asarray(x).reshape(-1))
        assert a.size == 2 * total * batch
        out = np.empty_like(a)
    elif kind == REAL_FORWARD:
        a = np.ascontiguousarray(np.asarray(x).reshape(-1), dtype=np.float64)
        assert a.size == total * batch
        out = np.empty(2 * htotal * batch, dtype=np.float64)
    else:
        a = _as_ri(np.asarray(x).reshape(-1))
        assert a.size == 2 * htotal * batch
        out = np.empty(total * batch, dtype=np.float64)
    ln = (ctypes.c_size_t * len(lengths))(*lengths)
    rc = _fn("orc_transform", ld)(ctypes.c_int(kind), ctypes.c_size_t(len(lengths)), ln,
                                  ctypes.c_size_t(batch), _dptr(a), _dptr(out))
    if rc != 0:
        raise ValueError("oracle rejected the transform description")
    return out if kind == REAL_INVERSE else out.view(np.complex128)


def rel_norms(a, b):
    """(relative L2, relative Linf) of a against reference b, over all scalars."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    if np.iscomplexobj(a) or np.iscomplexobj(b):
        a = a.astype(np.complex128).view(np.float64)
        b = b.astype(np.complex128).view(np.float64)
    a = np.ascontiguousarray(a, dtype=np.float64).reshape(-1)
    b = np.ascontiguousarray(b, dtype=np.float64).reshape(-1)
    assert a.size == b.size
    l2 = ctypes.c_double()
    li = ctypes.c_double()
    lib().orc_rel_norms_ld(_dptr(a), _dptr(b), ctypes.c_size_t(a.size), ctypes.byref(l2), ctypes.byref(li))
    return l2.value, li.value


def num_threads():
    return int(lib().orc_num_threads_d())
