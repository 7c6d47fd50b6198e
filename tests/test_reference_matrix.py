"""The reference's own accuracy-test matrix, run against the CPU checker through the C ABI.

The reference's rocfft-test generates its cases from the length lists of
clients/tests/accuracy_tests_range.h:41-164 (every 1D length from 2 to 8191, powers of 2, 3
and 5, radix-7/11/13 sizes, mixed sizes, primes, the stride lists), the ad-hoc sizes, layouts
and tokens of clients/tests/accuracy_test_adhoc.cpp:25-360 and the (length, stride, batch,
distance) tuples of clients/tests/accuracy_test_checkstride.cpp:26-100, and thins the cross
product by a hash of each case's token.  Here the length lists are walked in full with one
layout per transform kind and precision taken in rotation, so that every length and every
list entry is executed.  Length lists are written as the reference writes them (slowest
dimension first); rocfft.h takes the fastest first.

Tolerances: relative L2 and Linf <= 1e-5 in single and <= 1e-13 in double precision.
Lengths too long for a full comparison in seconds are checked on whole rows of a sample of
the batch, or on bins evaluated from the definition of the transform.
"""
import numpy as np
import pytest

import helpers as H
import inputs
import rocfft_amd.binding as B
from oracle import oracle as orc
from rocfft_amd.params import FFTParams

pytestmark = pytest.mark.gpu

# clients/tests/accuracy_tests_range.h:41-76
POW2_1D = [2 ** k for k in range(1, 31)]
POW3_1D = [3 ** k for k in range(1, 19)]
POW5_1D = [5 ** k for k in range(1, 13)]
RADX_1D = [7, 49, 84, 112, 11, 13, 52, 104, 208, 343, 2401, 16807]
MIX_1D = [6, 10, 12, 15, 20, 30, 56, 120, 150, 225, 240, 300, 336, 486, 600, 900, 1250, 1500, 1875, 2160, 2187,
          2250, 2500, 3000, 4000, 12000, 24000, 72000]
PRIME_1D = [17, 19, 23, 29, 31, 37, 41, 43, 47, 53, 59, 61, 67, 71, 73, 79, 83, 89, 97]
SMALL_1D_MAX = 8192  # small_1D_sizes(): every length from 2 below this (:79-104)
BATCH_1D = [4, 2, 1]  # :106
STRIDE_FOR_PRIME_1D = [1, 2, 3, 64, 65]  # :108-109
POW2_FOR_STRIDE_1D = [4096, 8192, 524288]  # :111
STRIDE_FOR_POW2_1D = [2, 3]  # :113
BATCH_FOR_STRIDE_1D = [2, 1]  # :114
# 2D and 3D lists (:121-164)
POW2_2D = [2, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048, 4096, 8192]
POW3_2D = [3, 9, 27, 81, 243, 729, 2187, 6561]
POW5_2D = [5, 25, 125, 625, 3125, 15625]
PRIME_2D = [7, 11, 13, 17, 19, 23, 29, 263, 269, 271, 277]
MIX_2D = [56, 120, 336, 2160, 5000, 6000, 8000]
POW2_3D = [4, 8, 16, 32, 128, 256]
POW3_3D = [3, 9, 27, 81, 243]
POW5_3D = [5, 25, 125]
PRIME_3D = [7, 11, 13, 17, 19, 23, 29]
SBRC_3D = [50, 64, 81, 100, 200, 10, 128, 256]
INNER_BATCH_3D = [4, 8, 16, 32, 20, 24, 64]

# the longest 1D transform compared element by element with the checker (it runs for seconds
# beyond); longer entries of the lists above are covered by test_long_lengths_of_the_1d_lists
FULL_COMPARE_MAX = 1 << 20


@pytest.fixture(scope="module")
def gpu(gpu_lib):
    return gpu_lib, H.TorchBackend()


def _tol(precision):
    return H.tolerance(precision)


class Sweep1D:
    """contiguous out-of-place 1D transforms of many lengths on one pair of device buffers"""

    def __init__(self, lib, be, kind, precision, max_elems):
        torch = be.torch
        self.lib, self.be, self.kind, self.precision = lib, be, kind, precision
        single = precision == B.SINGLE
        self.rt = np.float32 if single else np.float64
        self.ct = np.complex64 if single else np.complex128
        if kind == B.REAL_FORWARD:
            x = inputs.real_input(7001, 0, max_elems).astype(self.rt)
        else:
            x = inputs.complex_input(7002, 0, max_elems).astype(self.ct)
        self.x = x
        self.d_in = torch.from_numpy(x).to(be.dev)
        self.d_out = torch.empty(max_elems + 8, dtype=torch.complex64 if single else torch.complex128, device=be.dev)
        self.worst = (0.0, 0.0, None)

    def run(self, n, batch):
        torch = self.be.torch
        plan = B.Plan(B.NOTINPLACE, self.kind, self.precision, [n], batch, lib=self.lib)
        nout = n // 2 + 1 if self.kind == B.REAL_FORWARD else n
        self.d_out[:batch * nout + 8].fill_(float("nan"))
        plan.execute([self.d_in.data_ptr()], [self.d_out.data_ptr()])
        torch.cuda.synchronize()
        got = self.d_out[:batch * nout + 8].cpu().numpy()
        plan.destroy()
        assert np.isnan(got[batch * nout:].real).all(), ("wrote past the output", n, batch)
        xin = self.x[:batch * n].astype(np.float64 if self.kind == B.REAL_FORWARD else np.complex128)
        ref = orc.transform(self.kind, [n], batch, xin.reshape(batch, n), ld=self.precision == B.DOUBLE)
        l2, linf = orc.rel_norms(got[:batch * nout].astype(np.complex128), ref.reshape(-1))
        if not (l2 <= self.worst[0] and linf <= self.worst[1]):
            self.worst = (max(l2, self.worst[0]), max(linf, self.worst[1]), n)
        tol = _tol(self.precision)
        assert l2 <= tol and linf <= tol, (self.kind, n, batch, self.precision, l2, linf)


def test_every_1d_length_below_8192_complex_single(gpu):
    """small_1D_sizes() plus the lengths it leaves to the other lists: every n in [2, 8192)"""
    lib, be = gpu
    sw = Sweep1D(lib, be, B.COMPLEX_FORWARD, B.SINGLE, 4 * SMALL_1D_MAX)
    for n in range(2, SMALL_1D_MAX):
        if n % 1024 == 2:
            print("complex single n =", n, flush=True)
        sw.run(n, BATCH_1D[n % 3])
    print("worst (l2, linf, n)", sw.worst, flush=True)


def test_every_1d_length_below_8192_real_double(gpu):
    lib, be = gpu
    sw = Sweep1D(lib, be, B.REAL_FORWARD, B.DOUBLE, 4 * SMALL_1D_MAX)
    for n in range(2, SMALL_1D_MAX):
        if n % 1024 == 2:
            print("real double n =", n, flush=True)
        sw.run(n, BATCH_1D[(n + 1) % 3])
    print("worst (l2, linf, n)", sw.worst, flush=True)


KINDS = [B.COMPLEX_FORWARD, B.COMPLEX_INVERSE, B.REAL_FORWARD, B.REAL_INVERSE]


def _rotation(i):
    """(kind, precision, in place) taken in rotation over a list, so that a list as a whole meets
    every transform kind in both precisions and both placements"""
    return KINDS[i % 4], (B.SINGLE, B.DOUBLE)[(i // 4 + i) % 2], bool((i // 2) % 2)


@pytest.mark.parametrize("name", ["pow2", "pow3", "pow5", "radX", "mix", "prime"])
def test_1d_lists(gpu, name):
    lib, be = gpu
    lengths = dict(pow2=POW2_1D, pow3=POW3_1D, pow5=POW5_1D, radX=RADX_1D, mix=MIX_1D, prime=PRIME_1D)[name]
    i = 0
    for n in lengths:
        if n > FULL_COMPARE_MAX:
            continue
        for rep in range(2):  # two (kind, precision, placement) combinations per length
            kind, prec, inplace = _rotation(i)
            batch = BATCH_1D[i % 3] if n <= (1 << 16) else 1
            print(name, n, kind, prec, inplace, batch, flush=True)
            H.check(lib, be, kind, [n], batch, prec, inplace=inplace)
            i += 1


def test_prime_lengths_with_strides(gpu):
    """stride_range_for_prime_1D x prime_range_1D: the same stride on both sides"""
    lib, be = gpu
    i = 0
    for n in PRIME_1D:
        for s in STRIDE_FOR_PRIME_1D:
            kind, prec, inplace = _rotation(i)
            if kind in (B.REAL_FORWARD, B.REAL_INVERSE) and inplace:
                inplace = False  # (in-place real layouts tie the two strides together)
            batch = BATCH_1D[i % 3]
            nh = n // 2 + 1
            isz = nh if kind == B.REAL_INVERSE else n
            osz = nh if kind == B.REAL_FORWARD else n
            dist = max(isz, osz) * s + 3
            H.check(lib, be, kind, [n], batch, prec, inplace=inplace, in_strides=[s], in_dist=dist, out_strides=[s],
                    out_dist=dist)
            i += 1


def test_pow2_lengths_with_strides(gpu):
    """pow2_range_for_stride_1D x stride_range_for_pow2_1D x batch_range_for_stride_1D"""
    lib, be = gpu
    i = 0
    for n in POW2_FOR_STRIDE_1D:
        for s in STRIDE_FOR_POW2_1D:
            for batch in BATCH_FOR_STRIDE_1D:
                kind, prec, inplace = _rotation(i)
                if kind in (B.REAL_FORWARD, B.REAL_INVERSE):
                    inplace = False
                dist = n * s + 1
                print("stride", n, s, batch, kind, prec, inplace, flush=True)
                H.check(lib, be, kind, [n], batch, prec, inplace=inplace, in_strides=[s], in_dist=dist,
                        out_strides=[s], out_dist=dist)
                i += 1


def _rev(v):
    return list(reversed(v))


def test_2d_lists(gpu):
    """squares of the 2D lists plus neighbouring pairs (the reference takes the cross product and
    thins it); lengths whose square does not fit a full comparison in seconds pair with a short
    second dimension"""
    lib, be = gpu
    i = 0
    for lst in (POW2_2D, POW3_2D, POW5_2D, PRIME_2D, MIX_2D):
        for j, n in enumerate(lst):
            other = lst[(j + 1) % len(lst)]
            pairs = [[n, n], [n, other]]
            for ln in pairs:
                while ln[0] * ln[1] > (1 << 22):
                    ln[1] = max(2, ln[1] // 8)
                kind, prec, inplace = _rotation(i)
                print("2D", ln, kind, prec, inplace, flush=True)
                H.check(lib, be, kind, _rev(ln), 2 if ln[0] * ln[1] <= (1 << 20) else 1, prec, inplace=inplace)
                i += 1


def test_3d_lists(gpu):
    lib, be = gpu
    i = 0
    cases = []
    for lst in (POW2_3D, POW3_3D, POW5_3D, PRIME_3D):
        for j, n in enumerate(lst):
            cases.append([n, n, n])
            cases.append([n, lst[(j + 1) % len(lst)], lst[(j + 2) % len(lst)]])
    cases.append([4, 4, 8192])  # pow2_adhoc_3D
    for j, n in enumerate(SBRC_3D):  # sbrc_range_3D: cubes and mixed triples
        cases.append([n, SBRC_3D[(j + 3) % len(SBRC_3D)], SBRC_3D[(j + 5) % len(SBRC_3D)]])
    for j, n in enumerate(INNER_BATCH_3D):  # inner_batch_3D_range: small 2D slices, batched
        cases.append([INNER_BATCH_3D[(j + 2) % len(INNER_BATCH_3D)], n, n])
    for ln in cases:
        while ln[0] * ln[1] * ln[2] > (1 << 22):
            ln[0] = max(2, ln[0] // 4)
        kind, prec, inplace = _rotation(i)
        batch = (3, 2, 1)[i % 3] if ln[0] * ln[1] * ln[2] <= (1 << 18) else 1
        print("3D", ln, kind, prec, inplace, batch, flush=True)
        H.check(lib, be, kind, _rev(ln), batch, prec, inplace=inplace)
        i += 1


# Lengths of the 1D lists beyond FULL_COMPARE_MAX, and what the planner answers for those it
# cannot take (rocfft_plan_create returns rocfft_status_failure for them): none of the lists'
# entries today.  Each is run forward and back in one precision (the other in rotation): bins
# from the definition, Parseval and the round trip; a pure tone and a single impulse, whose
# transforms are known at every bin, check every output position.
REFUSED_1D = {}  # length -> status


def _closed_forms_1d(lib, be, n, precision):
    """x = impulse at n0 -> X_k = e^{-2 pi i k n0/n} at every k; x = e^{2 pi i k0 j/n} -> n at bin k0,
    0 elsewhere (phases reduced exactly in integers, evaluated in double precision on the device)"""
    torch = be.torch
    single = precision == B.SINGLE
    ct = torch.complex64 if single else torch.complex128
    tol = _tol(precision)
    fwd = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, precision, [n], 1, lib=lib)
    info = B.ExecutionInfo(lib)
    wb = fwd.work_buffer_size
    if wb:
        work = torch.empty(wb, dtype=torch.uint8, device=be.dev)
        info.set_work_buffer(work.data_ptr(), wb)
    x = torch.zeros(n, dtype=ct, device=be.dev)
    y = torch.empty(n, dtype=ct, device=be.dev)
    n0 = (n // 3) | 1
    x[n0] = 1.0
    fwd.execute([x.data_ptr()], [y.data_ptr()], info)
    torch.cuda.synchronize()
    worst = 0.0
    chunk = 1 << 24
    for lo in range(0, n, chunk):
        k = torch.arange(lo, min(n, lo + chunk), dtype=torch.int64, device=be.dev)
        ph = ((k * n0) % n).double() * (-2.0 * np.pi / n)
        d = torch.view_as_real(y[lo:lo + chunk]).double() - torch.stack([torch.cos(ph), torch.sin(ph)], -1)
        worst = max(worst, d.abs().max().item())
    assert worst <= tol * max(1.0, np.log2(n) / 8), ("impulse", n, worst)
    k0 = (2 * n // 7) | 1
    for lo in range(0, n, chunk):
        j = torch.arange(lo, min(n, lo + chunk), dtype=torch.int64, device=be.dev)
        ph = ((j * k0) % n).double() * (2.0 * np.pi / n)
        x[lo:lo + chunk] = torch.complex(torch.cos(ph), torch.sin(ph)).to(ct)
    fwd.execute([x.data_ptr()], [y.data_ptr()], info)
    torch.cuda.synchronize()
    peak = complex(y[k0].item())
    assert abs(peak - n) / n <= tol, ("tone", n, peak)
    y[k0] = 0
    rest = torch.view_as_real(y).abs().max().item()
    # every other bin is zero up to rounding: relative to the peak, as the norms of the comparison are
    assert rest / n <= tol, ("tone, other bins", n, rest / n)
    fwd.destroy()


LONG_1D = [n for n in POW2_1D + POW3_1D + POW5_1D + RADX_1D + MIX_1D if n > FULL_COMPARE_MAX]


@pytest.mark.parametrize("n", LONG_1D)
def test_long_lengths_of_the_1d_lists(gpu, n):
    lib, be = gpu
    i = LONG_1D.index(n)
    precision = (B.SINGLE, B.DOUBLE)[i % 2]
    if n >= (1 << 29):
        precision = B.SINGLE  # (2^29 and 2^30 in double precision: 8 and 16 GiB a buffer, not run here)
    if n in REFUSED_1D:
        with pytest.raises(B.RocfftError) as err:
            B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, precision, [n], 1, lib=lib)
        assert err.value.status == REFUSED_1D[n]
        return
    print("long", n, precision, flush=True)
    _spot_check_1d(lib, be, n, precision)
    be.torch.cuda.empty_cache()
    _closed_forms_1d(lib, be, n, precision)
    be.torch.cuda.empty_cache()


def test_prime_above_2_to_the_25(gpu):
    """33554467, the first prime above 2^25: its convolution length, 2^27, is beyond two levels of
    kernels (the reference takes any prime that fits memory, library/src/tree_node_bluestein.cpp:27-285);
    planned as 64 x 512 x 4096 with one launch of the row kernel per block of 512 rows"""
    lib, be = gpu
    n = 33554467
    print("prime", n, flush=True)
    _spot_check_1d(lib, be, n, B.SINGLE)
    be.torch.cuda.empty_cache()
    _closed_forms_1d(lib, be, n, B.SINGLE)
    be.torch.cuda.empty_cache()


# clients/tests/accuracy_test_adhoc.cpp:25-60 (slowest dimension first)
ADHOC_SIZES = [[1, 220], [1, 330], [81, 220, 36], [4, 4, 8192], [192, 192, 192], [192, 84, 84], [680, 128, 128],
               [196597], [25165813], [19, 2053], [98, 98, 98], [336, 336, 56]]


CHUNK = 1 << 24


def _device_bin(torch, x, k, direction):
    """bin k of the transform of the complex device vector x, from the definition: the phase
    j k mod n is reduced exactly in 64-bit integers, the terms are summed in double precision"""
    n = x.numel()
    re = im = 0.0
    for lo in range(0, n, CHUNK):
        j = torch.arange(lo, min(n, lo + CHUNK), dtype=torch.int64, device=x.device)
        ph = ((j * k) % n).double() * (direction * 2.0 * np.pi / n)
        c, s_ = torch.cos(ph), torch.sin(ph)
        xr = torch.view_as_real(x[lo:lo + CHUNK]).double()
        re += (xr[:, 0] * c - xr[:, 1] * s_).sum().item()
        im += (xr[:, 0] * s_ + xr[:, 1] * c).sum().item()
    return complex(re, im)


def _sumsq(torch, x):
    return sum(torch.view_as_real(x[lo:lo + CHUNK]).double().pow(2).sum().item() for lo in range(0, x.numel(), CHUNK))


def _absmax(torch, x):
    return max(torch.view_as_real(x[lo:lo + CHUNK]).abs().max().item() for lo in range(0, x.numel(), CHUNK))


def _spot_check_1d(lib, be, n, precision, kind=B.COMPLEX_FORWARD):
    """one long 1D complex transform: bins from the definition of the transform (on the host in
    long double up to 2^24 points, beyond that on the device in double precision), Parseval, and
    the unnormalised round trip"""
    torch = be.torch
    single = precision == B.SINGLE
    ct = torch.complex64 if single else torch.complex128
    x = torch.empty(n, dtype=ct, device=be.dev)
    for lo in range(0, n, CHUNK):
        m = min(CHUNK, n - lo)
        u = inputs.torch_uniform01(torch, be.dev, 7100 + n % 97, 2 * lo, 2 * m) - 0.5
        x[lo:lo + m] = torch.view_as_complex((u.to(torch.float32) if single else u).reshape(m, 2).contiguous())
        del u
    y = torch.empty_like(x)
    direction = -1 if kind == B.COMPLEX_FORWARD else +1

    def run(plan, src, dst):
        info = B.ExecutionInfo(lib)
        wb = plan.work_buffer_size
        work = torch.empty(max(wb, 1), dtype=torch.uint8, device=be.dev)
        if wb:
            info.set_work_buffer(work.data_ptr(), wb)
        plan.execute([src.data_ptr()], [dst.data_ptr()], info)
        torch.cuda.synchronize()

    fwd = B.Plan(B.NOTINPLACE, kind, precision, [n], 1, lib=lib)
    run(fwd, x, y)
    fwd.destroy()
    tol = _tol(precision)
    scale = _absmax(torch, y)
    xh = x.cpu().numpy().astype(np.complex128) if n <= (1 << 24) else None
    for k in (0, 1, n // 3, n // 2, n - 1):
        want = orc.dft_bin(xh, k, direction=direction) if xh is not None else _device_bin(torch, x, k, direction)
        got = complex(y[k].item())
        assert abs(got - want) / scale < tol, (n, k, got, want)
    del xh
    ex, ey = _sumsq(torch, x), _sumsq(torch, y)
    assert abs(ey / (n * ex) - 1.0) < 10 * tol, (n, ey / (n * ex))
    back = torch.empty_like(x)
    inv = B.Plan(B.NOTINPLACE, B.COMPLEX_INVERSE if kind == B.COMPLEX_FORWARD else B.COMPLEX_FORWARD, precision, [n], 1,
                 lib=lib)
    run(inv, y, back)
    inv.destroy()
    del y
    num = worst = 0.0
    for lo in range(0, n, CHUNK):
        d = torch.view_as_real(back[lo:lo + CHUNK]).double() / n - torch.view_as_real(x[lo:lo + CHUNK]).double()
        num += d.pow(2).sum().item()
        worst = max(worst, d.abs().max().item())
    l2 = (num / ex) ** 0.5
    li = worst / _absmax(torch, x)
    assert l2 <= tol and li <= 2 * tol, (n, l2, li)


@pytest.mark.parametrize("size", ADHOC_SIZES, ids=lambda s: "x".join(map(str, s)))
def test_adhoc_sizes(gpu, size):
    lib, be = gpu
    total = int(np.prod(size))
    if len(size) == 1 and total > FULL_COMPARE_MAX:
        _spot_check_1d(lib, be, size[0], B.DOUBLE)
        return
    big = total > (1 << 20)
    for i in range(1 if big else 8):
        kind, prec, inplace = _rotation(i + (len(size) + size[-1]) % 4)
        batch = 1 if big else BATCH_1D[i % 3]
        print("adhoc", size, kind, prec, inplace, batch, flush=True)
        H.check(lib, be, kind, _rev(size), batch, prec, inplace=inplace)


def test_adhoc_distances_are_ignored_for_one_transform(gpu):
    """param_permissive_iodist (accuracy_test_adhoc.cpp:84-157): in place, one transform,
    different input and output distances"""
    lib, be = gpu
    for i, size in enumerate([[4], [1, 220], [19, 2053], [98, 98, 98], [4, 4, 8192]]):
        kind, prec = KINDS[i % 2], (B.SINGLE, B.DOUBLE)[i % 2]
        H.check(lib, be, kind, _rev(size), 1, prec, inplace=True, in_dist=2, out_dist=3)


def test_adhoc_column_major(gpu):
    """param_adhoc_colmajor (:159-204): lengths and strides reversed, so that the first length
    has the longest stride (for real transforms all but the fastest dimension)"""
    lib, be = gpu
    for i, size in enumerate([[1, 220], [81, 220, 36], [4, 4, 8192], [192, 84, 84], [19, 2053], [98, 98, 98],
                              [336, 336, 56]]):
        kind = (B.COMPLEX_FORWARD, B.COMPLEX_INVERSE, B.REAL_FORWARD, B.REAL_INVERSE)[i % 4]
        real = kind in (B.REAL_FORWARD, B.REAL_INVERSE)
        if real and len(size) == 2:
            kind, real = B.COMPLEX_FORWARD, False
        p = FFTParams(kind, size, B.SINGLE, B.NOTINPLACE, 2).validate()
        keep = 1 if real else 0  # dimensions at the fast end that stay where they are
        cut = len(size) - keep
        length = _rev(p.length[:cut]) + p.length[cut:]
        istride = _rev(p.istride[:cut]) + p.istride[cut:]
        ostride = _rev(p.ostride[:cut]) + p.ostride[cut:]
        print("colmajor", length, istride, ostride, kind, flush=True)
        H.check(lib, be, kind, _rev(length), 2, B.SINGLE, in_strides=_rev(istride), in_dist=p.idist,
                out_strides=_rev(ostride), out_dist=p.odist)


def test_adhoc_strides(gpu):
    """param_adhoc_stride (:206-330)"""
    lib, be = gpu
    for prec in (B.SINGLE, B.DOUBLE):
        for inplace in (True, False):
            for it, ot in ((B.COMPLEX_INTERLEAVED, B.COMPLEX_INTERLEAVED), (B.COMPLEX_PLANAR, B.COMPLEX_PLANAR)) \
                    + (() if inplace else ((B.COMPLEX_INTERLEAVED, B.COMPLEX_PLANAR),
                                            (B.COMPLEX_PLANAR, B.COMPLEX_INTERLEAVED))):
                H.check(lib, be, B.COMPLEX_FORWARD, [35, 2], 2, prec, inplace=inplace, in_type=it, out_type=ot,
                        in_strides=[2, 90], in_dist=200, out_strides=[2, 90], out_dist=200)
        for ot in (B.HERMITIAN_INTERLEAVED, B.HERMITIAN_PLANAR):
            # (the reference gives both sides the same strides and lets validate() fix the distances)
            H.check(lib, be, B.REAL_FORWARD, [4, 4, 4], 2, prec, out_type=ot, in_strides=[1, 4, 16], in_dist=64,
                    out_strides=[1, 4, 16], out_dist=64)
            H.check(lib, be, B.REAL_FORWARD, [2, 2, 2], 2, prec, out_type=ot, in_strides=[1, 6, 20], in_dist=40,
                    out_strides=[1, 6, 20], out_dist=40)


# accuracy_test_adhoc.cpp:337-352
ADHOC_TOKENS = [
    "complex_forward_len_4_4_4_single_op_batch_2_istride_16_4_1_CI_ostride_4_16_1_CI_idist_64_odist_64_ioffset_0_0_ooffset_0_0",
    "complex_forward_len_512_64_single_ip_batch_3_istride_192_3_CI_ostride_192_3_CI_idist_1_odist_1_ioffset_0_0_ooffset_0_0",
    "real_forward_len_1024_1024_1024_single_op_batch_1_istride_1048576_1024_1_R_ostride_525312_513_1_HI_idist_1073741824_odist_537919488_ioffset_0_0_ooffset_0_0",
    "complex_forward_len_6144_single_ip_batch_34_istride_35_CI_ostride_35_CI_idist_1_odist_1_ioffset_0_0_ooffset_0_0",
    "real_forward_len_8192_single_ip_batch_65537_istride_1_R_ostride_1_HI_idist_8194_odist_4097_ioffset_0_0_ooffset_0_0",
    "real_forward_len_520_single_op_batch_270400_istride_1_R_ostride_1_HI_idist_520_odist_261_ioffset_0_0_ooffset_0_0",
    "real_forward_len_630_single_op_batch_396900_istride_1_R_ostride_1_HI_idist_630_odist_316_ioffset_0_0_ooffset_0_0",
    "real_forward_len_660_single_op_batch_435600_istride_1_R_ostride_1_HI_idist_660_odist_331_ioffset_0_0_ooffset_0_0",
    "real_forward_len_700_single_op_batch_490000_istride_1_R_ostride_1_HI_idist_700_odist_351_ioffset_0_0_ooffset_0_0",
    "real_forward_len_728_single_op_batch_529984_istride_1_R_ostride_1_HI_idist_728_odist_365_ioffset_0_0_ooffset_0_0",
    "real_forward_len_968_single_op_batch_937024_istride_1_R_ostride_1_HI_idist_968_odist_485_ioffset_0_0_ooffset_0_0",
    "real_forward_len_1020_single_op_batch_1040400_istride_1_R_ostride_1_HI_idist_1020_odist_511_ioffset_0_0_ooffset_0_0",
]


def _run_token_sampled(lib, be, token, sample=24):
    """A token of the default (or in-place padded) 1D real layout with a very large batch: the
    whole batch runs, a sample of its rows is compared with the checker."""
    torch = be.torch
    p = FFTParams.from_token(token).validate()
    assert p.transform_type == B.REAL_FORWARD and len(p.length) == 1 and p.precision == B.SINGLE
    n, batch, nh = p.length[0], p.nbatch, p.length[0] // 2 + 1
    inplace = p.placement == B.INPLACE
    x = (inputs.torch_uniform01(torch, be.dev, 7200 + n, 0, batch * p.idist) * 2.0 - 1.0).to(torch.float32)
    keep = x.clone()
    rows = np.unique(np.concatenate([[0, 1, batch - 1], (inputs.uniform01(7300 + n, 0, sample) * batch).astype(np.int64)]))
    xin = x.reshape(batch, p.idist)[torch.from_numpy(rows).to(be.dev), :n].cpu().numpy().astype(np.float64)
    plan = p.make_plan(lib)
    if inplace:
        assert p.idist == 2 * p.odist
        plan.execute([x.data_ptr()], None)
        out = torch.view_as_complex(x.reshape(batch, p.odist, 2))
    else:
        out = torch.full((batch, p.odist), float("nan"), dtype=torch.complex64, device=be.dev)
        plan.execute([x.data_ptr()], [out.data_ptr()])
    torch.cuda.synchronize()
    got = out[torch.from_numpy(rows).to(be.dev), :nh].cpu().numpy().astype(np.complex128)
    ref = orc.transform(orc.REAL_FORWARD, [n], len(rows), xin)
    l2, linf = orc.rel_norms(got.reshape(-1), ref.reshape(-1))
    assert l2 <= 1e-5 and linf <= 1e-5, (token, l2, linf)
    # every row: finite, and Parseval per row against the input (sum |X_k|^2 over the full
    # spectrum = n sum x^2; the stored half counts bins 1 .. (n-1)/2 twice)
    o = out[:, :nh]
    w = torch.full((nh,), 2.0, dtype=torch.float64, device=be.dev)
    w[0] = 1.0
    if n % 2 == 0:
        w[nh - 1] = 1.0
    ey = (torch.view_as_real(o).double().pow(2).sum(-1) * w).sum(-1)
    ex = keep.reshape(batch, p.idist)[:, :n].double().pow(2).sum(-1) * n
    assert torch.isfinite(ey).all()
    assert ((ey / ex - 1.0).abs().max().item()) < 1e-4, token
    if not inplace:
        assert torch.equal(x, keep)
    plan.destroy()


@pytest.mark.parametrize("token", ADHOC_TOKENS, ids=lambda t: t.split("_single")[0])
def test_adhoc_tokens(gpu, token):
    lib, be = gpu
    p = FFTParams.from_token(token).validate()
    total = int(np.prod(p.length)) * p.nbatch
    if total <= (1 << 21):
        from test_tokens import run_token
        run_token(lib, be, token)
    elif len(p.length) == 1:
        _run_token_sampled(lib, be, token)
    else:
        _check_real_cube_1024(lib, be, p)


def _check_real_cube_1024(lib, be, p):
    """real forward 1024^3, single precision (4 GiB in, 4 GiB out): bins from the definition
    along separable inputs are not available for random data, so the input is a sum of a few
    plane waves plus a point, whose transform is known in closed form at every bin"""
    torch = be.torch
    assert p.length == [1024, 1024, 1024] and p.transform_type == B.REAL_FORWARD
    n = 1024
    dev = be.dev
    i2 = torch.arange(n, device=dev, dtype=torch.float64).reshape(n, 1, 1)
    i1 = torch.arange(n, device=dev, dtype=torch.float64).reshape(1, n, 1)
    i0 = torch.arange(n, device=dev, dtype=torch.float64).reshape(1, 1, n)
    waves = [(3, 5, 7, 0.5), (1000, 17, 129, -0.25), (0, 0, 512, 0.125), (511, 512, 1, 0.75)]  # (k2, k1, k0, amp)
    x = torch.zeros((n, n, n), dtype=torch.float32, device=dev)
    for k2, k1, k0, a in waves:
        ph = ((i2 * k2 + i1 * k1 + i0 * k0) % n) * (2.0 * np.pi / n)
        x += (a * torch.cos(ph)).to(torch.float32)
        del ph
    point = (37, 901, 444)
    x[point] += 2.0
    out = torch.empty((n, n, n // 2 + 1), dtype=torch.complex64, device=dev)
    plan = p.make_plan(lib)
    info = B.ExecutionInfo(lib)
    wb = plan.work_buffer_size
    if wb:
        work = torch.empty(wb, dtype=torch.uint8, device=dev)
        info.set_work_buffer(work.data_ptr(), wb)
    plan.execute([x.data_ptr()], [out.data_ptr()], info)
    torch.cuda.synchronize()
    # expected: the point contributes 2 e^{-2 pi i (k . point)/n} everywhere; a cosine wave of
    # amplitude a contributes a n^3 / 2 at +-k (a n^3 when k = -k mod n)
    h = n // 2 + 1
    k0 = torch.arange(h, device=dev, dtype=torch.float64).reshape(1, 1, h)
    ph = ((i2 * point[0] + i1 * point[1] + k0 * point[2]) % n) * (-2.0 * np.pi / n)
    exp_re = 2.0 * torch.cos(ph)
    exp_im = 2.0 * torch.sin(ph)
    del ph
    total = float(n) ** 3
    for k2, k1, kk0, a in waves:
        for s in (1, -1):
            q2, q1, q0 = (s * k2) % n, (s * k1) % n, (s * kk0) % n
            selfconj = ((2 * k2) % n == 0 and (2 * k1) % n == 0 and (2 * kk0) % n == 0)
            if q0 < h and not (selfconj and s == -1):
                exp_re[q2, q1, q0] += a * total * (1.0 if selfconj else 0.5)
    d_re = out.real.double() - exp_re
    d_im = out.imag.double() - exp_im
    scale = 0.75 * total * 0.5
    linf = max(d_re.abs().max().item(), d_im.abs().max().item()) / scale
    l2 = ((d_re.pow(2).sum() + d_im.pow(2).sum()).sqrt() / (exp_re.pow(2).sum() + exp_im.pow(2).sum()).sqrt()).item()
    assert linf <= 1e-5 and l2 <= 1e-5, (l2, linf)
    plan.destroy()


# accuracy_test_checkstride.cpp:39-66: (lengths, strides, batch, distance), slowest dimension first
CHECKSTRIDE = [([64], [2], 2, 140), ([64], [1], 2, 80), ([15], [2], 2, 40), ([8192], [2], 2, 17000),
               ([24000], [2], 2, 50000), ([20, 30], [80, 2], 2, 1700), ([40, 30], [80, 2], 2, 3600),
               ([20, 30], [40, 1], 2, 1000), ([40, 30], [40, 1], 2, 2000), ([64, 64], [130, 2], 2, 8400),
               ([64, 64, 64], [8400, 130, 2], 2, 540000), ([2, 3, 4], [40, 10, 2], 2, 100),
               ([30, 40, 50], [3000, 60, 1], 2, 100000)]


@pytest.mark.parametrize("case", CHECKSTRIDE, ids=lambda c: "x".join(map(str, c[0])) + "_s" + "_".join(map(str, c[1])))
def test_checkstride(gpu, case):
    """out of place, the same strides and distance on both sides, the output buffer filled with a
    guard pattern beforehand: the result is right and every byte between its elements is left
    alone (the reference's check_output_strides, shared/accuracy_test.h:611-682).  All four
    transform kinds in both precisions; interleaved and planar complex sides in rotation; with
    load and store callbacks on the interleaved cases."""
    from test_callbacks import S_LOAD, S_STORE, callback_library, make_hook

    lib, be = gpu
    cblib = callback_library("libcb_device.so")
    lengths, strides, batch, dist = case
    i = 0
    for kind in KINDS:
        for prec in (B.SINGLE, B.DOUBLE):
            real_in, real_out = kind == B.REAL_FORWARD, kind == B.REAL_INVERSE
            planar = i % 3 == 2
            it = B.REAL if real_in else (B.HERMITIAN_PLANAR if real_out else B.COMPLEX_PLANAR) if planar else None
            ot = B.REAL if real_out else (B.HERMITIAN_PLANAR if real_in else B.COMPLEX_PLANAR) if planar else None
            for with_cb in ((False,) if planar else (False, True)):
                kw = dict(in_strides=_rev(strides), in_dist=dist, out_strides=_rev(strides), out_dist=dist)
                if it is not None:
                    kw.update(in_type=it, out_type=ot)
                if with_cb:
                    kw["info_hook"] = make_hook(cblib, kind, prec, "load+store")
                y, x, touched = H.run_transform(lib, be, kind, _rev(lengths), batch, prec, return_buffers=True, **kw)
                for raw, mask in touched:
                    assert np.all(raw[~mask[:raw.size]] == H.GUARD), ("stray write", case, kind, prec, planar, with_cb)
                ref = H.reference(kind, _rev(lengths), batch, x, prec) * (S_LOAD * S_STORE if with_cb else 1.0)
                l2, linf = orc.rel_norms(y.reshape(-1), ref.reshape(-1))
                tol = _tol(prec)
                assert l2 <= tol and linf <= tol, (case, kind, prec, planar, with_cb, l2, linf)
            i += 1
