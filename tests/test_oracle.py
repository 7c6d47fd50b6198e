"""Pins the CPU checker (oracle/) before anything is compared against it.

Every exported function of oracle/fft_oracle.c is checked against something it
does not share code with: the DFT definition and closed forms, brute force on
small sizes, numpy's pocketfft, and the committed golden fixtures.  A dropped
term, a wrong sign or index or a transposed operand fails at least one check.
"""
import os

import numpy as np
import pytest

import inputs
from oracle import oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL_LD = 5e-16  # long double build, results rounded to double
TOL_D = 5e-15  # double build


def rnd_c(n, seed=0):
    return inputs.complex_input(seed + 1, 0, n)


# ---------------------------------------------------------------- naive DFT
@pytest.mark.parametrize("n", [1, 2, 3, 8, 15, 64])
def test_naive_closed_forms(n):
    delta = np.zeros(n, dtype=complex)
    delta[0] = 1
    assert np.allclose(orc.dft_naive(delta), np.ones(n), atol=1e-15)
    const = np.ones(n, dtype=complex)
    want = np.zeros(n, dtype=complex)
    want[0] = n
    assert np.allclose(orc.dft_naive(const), want, atol=1e-13)
    for k0 in {0, 1, n // 2, n - 1}:
        x = np.exp(2j * np.pi * k0 * np.arange(n) / n)
        want = np.zeros(n, dtype=complex)
        want[k0 % n] = n
        assert np.allclose(orc.dft_naive(x), want, atol=1e-12 * n), (n, k0)
        # the inverse sign puts the spike at -k0
        want = np.zeros(n, dtype=complex)
        want[(-k0) % n] = n
        assert np.allclose(orc.dft_naive(x, +1), want, atol=1e-12 * n), (n, k0)


def test_naive_shift_theorem_and_numpy():
    n = 45
    x = rnd_c(n)
    X = orc.dft_naive(x)
    Xs = orc.dft_naive(np.roll(x, 3))
    assert np.allclose(Xs, X * np.exp(-2j * np.pi * 3 * np.arange(n) / n), atol=1e-13)
    assert orc.rel_norms(X, np.fft.fft(x))[0] < 1e-15
    assert orc.rel_norms(orc.dft_naive(x, +1), np.fft.ifft(x) * n)[0] < 1e-15


def test_dft_bin_matches_naive_and_numpy():
    n = 1009
    x = rnd_c(n, 3)
    X = np.fft.fft(x)
    for k in (0, 1, 500, 1008):
        assert abs(orc.dft_bin(x, k) - X[k]) < 1e-12
    # exact phase reduction for n*k beyond 2^53
    n = 1000003
    x = rnd_c(n, 4)
    X = np.fft.fft(x)
    for k in (1, 999983, 1000002):
        assert abs(orc.dft_bin(x, k) - X[k]) / np.abs(X).max() < 1e-13


# ---------------------------------------------------------------- Stockham
@pytest.mark.parametrize("factors", [[2], [4, 4], [16, 16, 16], [8, 8, 4, 4], [3, 5, 7], [5, 2, 3, 2],
                                     [13, 11], [17, 2], [16, 8]])
def test_stockham_vs_naive(factors):
    n = int(np.prod(factors))
    x = rnd_c(n, n)
    ref = orc.dft_naive(x) if n <= 2048 else np.fft.fft(x)
    tol = TOL_LD if n <= 2048 else 2e-15
    for d in (-1, +1):
        ref_d = ref if d < 0 else (orc.dft_naive(x, +1) if n <= 2048 else np.fft.ifft(x) * n)
        assert orc.rel_norms(orc.stockham(x, factors, d, ld=True), ref_d)[0] < tol
        assert orc.rel_norms(orc.stockham(x, factors, d, ld=False), ref_d)[0] < TOL_D


def test_stacked_twiddle_table_layout():
    # reference layout: T[off_p + j*(w-1) + k-1] = exp(-2 pi i jk/(c w)); 16x16x16 has 4080 entries
    t = orc.stacked_twiddles(4096, [16, 16, 16])
    assert t.size == 15 * 16 + 15 * 256
    c, w, off = 16, 16, 0
    for j, k in [(0, 1), (3, 5), (15, 15)]:
        assert abs(t[off + j * (w - 1) + k - 1] - np.exp(-2j * np.pi * j * k / (c * w))) < 1e-15
    c, off = 256, 15 * 16
    for j, k in [(1, 1), (200, 7), (255, 15)]:
        assert abs(t[off + j * (w - 1) + k - 1] - np.exp(-2j * np.pi * j * k / (c * w))) < 1e-15


def test_factorize():
    assert int(np.prod(orc.factorize(4096))) == 4096 and set(orc.factorize(4096)) == {16}
    assert sorted(orc.factorize(210)) == [2, 3, 5, 7]
    assert orc.factorize(97) == [] and orc.factorize(2 * 19) == []


# ---------------------------------------------------------------- fft1d (all routes)
@pytest.mark.parametrize("n", [1, 2, 6, 17, 19, 23, 29, 31, 37, 41, 43, 47, 53, 59, 61, 67, 71, 73, 79, 83,
                               89, 97, 128, 243, 625, 1000, 1024, 8191])
def test_fft1d_vs_naive(n):
    x = rnd_c(n, n)
    ref = orc.dft_naive(x)
    assert orc.rel_norms(orc.fft1d(x, ld=True), ref)[0] < 2e-16 * max(1, np.log2(n))
    assert orc.rel_norms(orc.fft1d(x, ld=False), ref)[0] < TOL_D
    assert orc.rel_norms(orc.fft1d(x, +1, ld=True), orc.dft_naive(x, +1))[0] < 2e-16 * max(1, np.log2(n))


@pytest.mark.parametrize("n", [4096, 32768, 65536, 1000003])
def test_fft1d_large_vs_numpy_and_bins(n):
    x = rnd_c(n, 11)
    y = orc.fft1d(x, ld=True)
    assert orc.rel_norms(y, np.fft.fft(x))[0] < 3e-16 * np.sqrt(np.log2(n))
    for k in (0, 1, n // 3, n - 1):
        assert abs(y[k] - orc.dft_bin(x, k)) / np.abs(y).max() < 1e-15
    # Parseval and linearity
    assert abs(np.vdot(y, y).real - n * np.vdot(x, x).real) / (n * np.vdot(x, x).real) < 1e-14
    z = rnd_c(n, 12)
    assert orc.rel_norms(orc.fft1d(x + 2j * z, ld=True), y + 2j * orc.fft1d(z, ld=True))[0] < 1e-15


@pytest.mark.parametrize("n", [5, 16, 17, 97, 360, 1009])
def test_bluestein_route_vs_naive(n):
    x = rnd_c(n, n + 5)
    for d in (-1, +1):
        assert orc.rel_norms(orc.bluestein1d(x, d, ld=True), orc.dft_naive(x, d))[0] < 1e-15
        assert orc.rel_norms(orc.bluestein1d(x, d, ld=False), orc.dft_naive(x, d))[0] < TOL_D


# ---------------------------------------------------------------- large 1D pieces
def test_large_twiddle_products():
    # the reference's table for 32768 = 128*256: base 5, 3 steps (library/src/plan.cpp:3296-3313)
    L = 32768
    for u in (0, 1, 31, 32, 1023, 1024, 32767, 127 * 255):
        w = orc.large_twiddle(L, 5, 3, u)
        assert abs(w - np.exp(-2j * np.pi * (u % L) / L)) < 4e-16
    assert abs(orc.large_twiddle(2 ** 21, 8, 3, 1234567) - np.exp(-2j * np.pi * 1234567 / 2 ** 21)) < 4e-16


@pytest.mark.parametrize("n1,n0,base,steps", [(128, 256, 5, 3), (8, 4, 3, 2), (12, 10, 4, 2), (64, 64, 6, 2)])
def test_large1d_cc_vs_direct(n1, n0, base, steps):
    x = rnd_c(n1 * n0, n1)
    for d in (-1, +1):
        ref = np.fft.fft(x) if d < 0 else np.fft.ifft(x) * x.size
        assert orc.rel_norms(orc.large1d_cc(x, n1, n0, base, steps, d), ref)[0] < 1e-15


# ---------------------------------------------------------------- real pre/post
@pytest.mark.parametrize("n", [2, 4, 6, 8, 10, 64, 250, 4096])
def test_r2c_post_and_c2r_pre(n):
    x = inputs.real_input(5, 0, n)
    z = x[0::2] + 1j * x[1::2]
    Z = np.fft.fft(z)
    X = orc.r2c_post(Z)
    assert X.size == n // 2 + 1
    assert orc.rel_norms(X, np.fft.rfft(x))[0] < 1e-15
    # pre-processing followed by the half-length inverse gives n*x as interleaved pairs
    zz = np.fft.ifft(orc.c2r_pre(X)) * (n // 2)
    back = np.empty(n)
    back[0::2], back[1::2] = zz.real, zz.imag
    assert orc.rel_norms(back, n * x)[0] < 1e-14
    # imaginary parts of the DC and Nyquist bins are ignored, bit for bit
    X2 = X.copy()
    X2[0] += 3j
    X2[-1] -= 7j
    assert np.array_equal(orc.c2r_pre(X2).view(np.float64), orc.c2r_pre(X).view(np.float64))


# ---------------------------------------------------------------- whole transforms
def np_forward(kind, lengths, batch, x):
    shape = (batch,) + tuple(reversed(lengths))
    axes = tuple(range(1, len(lengths) + 1))
    if kind == orc.COMPLEX_FORWARD:
        return np.fft.fftn(x.reshape(shape), axes=axes).reshape(-1)
    if kind == orc.COMPLEX_INVERSE:
        return np.fft.ifftn(x.reshape(shape), axes=axes, norm="forward").reshape(-1)
    if kind == orc.REAL_FORWARD:
        return np.fft.rfftn(x.reshape(shape), axes=axes).reshape(-1)
    h0 = lengths[0] // 2 + 1
    hshape = (batch,) + tuple(reversed(lengths[1:])) + (h0,)
    return np.fft.irfftn(x.reshape(hshape), s=tuple(reversed(lengths)), axes=axes, norm="forward").reshape(-1)


@pytest.mark.parametrize("lengths", [[8], [9], [30], [4096], [17], [16, 8], [9, 5], [12, 10, 6], [32, 8, 4],
                                     [7, 6, 5], [34, 3]])
@pytest.mark.parametrize("kind", [0, 1, 2, 3])
def test_transform_vs_numpy(kind, lengths, batch=3):
    total = int(np.prod(lengths))
    if kind in (0, 1):
        x = rnd_c(total * batch, total)
    elif kind == 2:
        x = inputs.real_input(8, 0, total * batch)
    else:
        x = np_forward(2, lengths, batch, inputs.real_input(8, 0, total * batch))
    for ld in (True, False):
        y = orc.transform(kind, lengths, batch, x, ld=ld)
        assert orc.rel_norms(y, np_forward(kind, lengths, batch, x))[0] < (1e-15 if ld else TOL_D)


def test_transform_roundtrip_is_unnormalised():
    lengths, batch = [10, 6, 4], 2
    total = 240
    x = inputs.real_input(9, 0, total * batch)
    back = orc.transform(3, lengths, batch, orc.transform(2, lengths, batch, x, ld=True), ld=True)
    assert orc.rel_norms(back, total * x)[0] < 1e-15


def test_rel_norms_formula():
    a = np.array([1.0, 2.0, 3.5])
    b = np.array([1.0, 2.5, 3.0])
    l2, linf = orc.rel_norms(a, b)
    assert abs(l2 - np.sqrt(0.5) / np.sqrt(1 + 6.25 + 9)) < 1e-15
    assert abs(linf - 0.5 / 3.0) < 1e-15


# ---------------------------------------------------------------- golden fixtures
@pytest.mark.parametrize("cfg_id", [1, 2, 3, 4, 5])
def test_oracle_matches_golden_fixture(cfg_id):
    g = np.load(os.path.join(GOLDEN, "cfg%d.npz" % cfg_id))
    rows = 1 if cfg_id in (3, 4) else int(g["rows"])
    c = inputs.CONFIGS[cfg_id]
    x = inputs.config_input(cfg_id, 0, rows)
    assert np.array_equal(x[:, :4], g["input_head"][:rows])
    kind = orc.COMPLEX_FORWARD if c["kind"] == "c2c" else orc.REAL_FORWARD
    # long double for the sizes where that takes seconds, double for the two big ones
    y = orc.transform(kind, c["lengths"], rows, x, ld=cfg_id not in (3, 4)).reshape(rows, -1)
    scale = g["l2"][:rows, None] / np.sqrt(y.shape[1])  # rms magnitude of a bin
    assert np.max(np.abs(y[:, g["bins"]] - g["values"][:rows]) / scale) < 1e-13
    assert np.max(np.abs(y.sum(axis=1) - g["total"][:rows]) / (scale[:, 0] * np.sqrt(y.shape[1]))) < 1e-12
    assert np.max(np.abs(np.sqrt((np.abs(y) ** 2).sum(axis=1)) / g["l2"][:rows] - 1)) < 1e-13
