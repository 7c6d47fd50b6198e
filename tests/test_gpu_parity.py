"""GPU parity tests: the HIP library, called through its C ABI, against the CPU
checker on the same seeded inputs, against the committed golden fixtures, and --
at the full benchmark sizes -- through size-independent properties (unnormalised
round trip, Parseval, spot bins evaluated from the DFT definition) plus a
cross-check against torch.fft, which on ROCm is the reference rocFFT behind
hipFFT.

Tolerances are the north-star bar: relative L2 and Linf <= 1e-5 in single and
<= 1e-13 in double precision (helpers.tolerance).
"""
import os
import threading

import numpy as np
import pytest

import helpers as H
import inputs
import rocfft_amd.binding as B
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def gpu(gpu_lib):
    return gpu_lib, H.TorchBackend()


def tnorm(torch, a, b):
    """(rel L2, rel Linf) of a against b, both device tensors, over all scalars"""
    a = torch.view_as_real(a) if a.is_complex() else a
    b = torch.view_as_real(b) if b.is_complex() else b
    d = (a.double() - b.double())
    l2 = (torch.linalg.vector_norm(d) / torch.linalg.vector_norm(b.double())).item()
    li = (d.abs().max() / b.double().abs().max()).item()
    return l2, li


# ------------------------------------------------------------------ against the checker
@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 7, 8, 9, 16, 30, 64, 100, 128, 256, 512, 1000, 1024, 2048, 4096,
                               8192, 11, 13, 17, 97, 121, 1001, 2310])
def test_c2c_1d(gpu, n):
    lib, be = gpu
    for prec in (B.SINGLE, B.DOUBLE):
        H.check(lib, be, B.COMPLEX_FORWARD, [n], 5, prec)
        H.check(lib, be, B.COMPLEX_INVERSE, [n], 3, prec, inplace=True)


@pytest.mark.parametrize("n", [2, 4, 6, 8, 30, 64, 256, 1000, 4096, 8192, 3, 9, 15, 17, 34, 97, 194])
def test_real_1d(gpu, n):
    lib, be = gpu
    for prec in (B.SINGLE, B.DOUBLE):
        for kind in (B.REAL_FORWARD, B.REAL_INVERSE):
            H.check(lib, be, kind, [n], 5, prec)
            H.check(lib, be, kind, [n], 2, prec, inplace=True)


def test_every_compiled_schedule(gpu):
    """Each length with a compile-time-schedule kernel: complex both directions, and the real
    transforms of twice the length (whose half-length complex transform is that kernel with the
    fused pre/post-processing, odd lengths included)."""
    lib, be = gpu
    for n, radix, tf, td in H.fast_schedules():
        print("schedule", n, radix, flush=True)
        H.check(lib, be, B.COMPLEX_FORWARD, [n], 5, B.SINGLE)
        H.check(lib, be, B.COMPLEX_INVERSE, [n], 3, B.DOUBLE, inplace=True)
        H.check(lib, be, B.REAL_FORWARD, [2 * n], 3, B.SINGLE)
        H.check(lib, be, B.REAL_INVERSE, [2 * n], 3, B.DOUBLE)
        if n % 2 == 1:
            # odd-length real transforms run the same kernel with real samples on one side
            H.check(lib, be, B.REAL_FORWARD, [n], 3, B.DOUBLE)
            H.check(lib, be, B.REAL_INVERSE, [n], 3, B.SINGLE)


def test_odd_real_layouts(gpu):
    """Odd-length real transforms in one kernel: in place (padded rows), strided real side, a
    scale factor, as dimension 0 of 2D/3D transforms, planar bins (no compiled variant: the
    generic kernel), and a misaligned complex side."""
    lib, be = gpu
    for n in (9, 77, 153, 625, 1001, 2187, 4095):
        H.check(lib, be, B.REAL_FORWARD, [n], 4, B.SINGLE, inplace=True, scale=0.5)
        H.check(lib, be, B.REAL_INVERSE, [n], 4, B.DOUBLE, inplace=True, scale=0.25)
        H.check(lib, be, B.REAL_FORWARD, [n], 3, B.DOUBLE, in_strides=[3], in_dist=3 * n + 1)
        H.check(lib, be, B.REAL_INVERSE, [n], 3, B.SINGLE, out_strides=[2], out_dist=2 * n + 3)
        H.check(lib, be, B.REAL_FORWARD, [n], 2, B.SINGLE, out_type=B.HERMITIAN_PLANAR)
        H.check(lib, be, B.REAL_INVERSE, [n], 2, B.DOUBLE, in_type=B.HERMITIAN_PLANAR)
        H.check(lib, be, B.REAL_FORWARD, [n], 2, B.SINGLE, in_offsets=[1, 0], out_offsets=[3, 0])
        H.check(lib, be, B.REAL_INVERSE, [n], 2, B.SINGLE, in_offsets=[5, 0], out_offsets=[1, 0])
    for lengths in ([7, 33, 5], [77, 27], [429, 64], [175, 35, 6], [25, 25, 25], [135, 512]):
        for prec in (B.SINGLE, B.DOUBLE):
            H.check(lib, be, B.REAL_FORWARD, lengths, 3, prec)
            H.check(lib, be, B.REAL_INVERSE, lengths, 3, prec)
    # lengths with a large prime factor: the chirp-z convolution in one kernel, real samples on one side
    for n in (17, 173, 1009, 2849):
        for prec in (B.SINGLE, B.DOUBLE):
            H.check(lib, be, B.REAL_FORWARD, [n], 5, prec)
            H.check(lib, be, B.REAL_INVERSE, [n], 5, prec)
        H.check(lib, be, B.REAL_FORWARD, [n], 4, B.SINGLE, inplace=True, scale=0.5)
        H.check(lib, be, B.REAL_INVERSE, [n], 4, B.DOUBLE, inplace=True, scale=0.25)
        H.check(lib, be, B.REAL_FORWARD, [n], 3, B.DOUBLE, in_strides=[3], in_dist=3 * n + 1)
        H.check(lib, be, B.REAL_INVERSE, [n], 3, B.SINGLE, out_strides=[2], out_dist=2 * n + 3)
        H.check(lib, be, B.REAL_FORWARD, [n], 2, B.SINGLE, in_offsets=[1, 0], out_offsets=[3, 0])
        H.check(lib, be, B.REAL_INVERSE, [n], 2, B.SINGLE, in_offsets=[5, 0], out_offsets=[1, 0])
    for lengths in ([173, 14, 27], [2849, 9], [97, 97]):
        for prec in (B.SINGLE, B.DOUBLE):
            H.check(lib, be, B.REAL_FORWARD, lengths, 3, prec)
            H.check(lib, be, B.REAL_INVERSE, lengths, 3, prec)


def test_compiled_schedules_in_other_layouts(gpu):
    """Strided, planar and column uses of non-power-of-two schedules: column passes of the
    compiled kernel, and the generic kernel on the same schedule where the layout has no
    compiled variant."""
    lib, be = gpu
    K = B
    for n in (100, 243, 1000, 3000):
        H.check(lib, be, K.COMPLEX_FORWARD, [n], 3, K.SINGLE, in_type=K.COMPLEX_PLANAR, out_type=K.COMPLEX_PLANAR)
        H.check(lib, be, K.COMPLEX_INVERSE, [n], 3, K.DOUBLE, in_strides=[3], in_dist=3 * n + 5, out_strides=[2],
                out_dist=2 * n + 1)
        H.check(lib, be, K.COMPLEX_FORWARD, [n], 8, K.SINGLE, in_strides=[8], in_dist=1, out_strides=[8], out_dist=1)
        H.check(lib, be, K.REAL_FORWARD, [2 * n], 3, K.DOUBLE, out_type=K.HERMITIAN_PLANAR)
        H.check(lib, be, K.COMPLEX_FORWARD, [n], 2, K.DOUBLE, scale=0.125)
    for lengths in ([100, 100], [60, 90], [9, 10, 6], [1000, 12], [12, 1000], [360, 360]):
        for kind in (K.COMPLEX_FORWARD, K.REAL_FORWARD, K.REAL_INVERSE):
            H.check(lib, be, kind, lengths, 2, K.SINGLE)
            H.check(lib, be, kind, lengths, 2, K.DOUBLE, inplace=(kind == K.COMPLEX_FORWARD))
    for n in (5000, 6000, 9000, 10000, 6561, 100000):
        H.check(lib, be, K.COMPLEX_FORWARD, [n], 2, K.SINGLE)
        H.check(lib, be, K.REAL_INVERSE, [n], 2, K.DOUBLE)


def test_planar_arrays_on_the_compiled_kernels(gpu):
    """Planar complex and Hermitian arrays (real and imaginary parts in separate buffers) take the
    compiled kernels like interleaved ones: every fused operation of that path (plain passes,
    Hermitian pre/post-processing of even lengths, odd-length real transforms, the Bluestein chirp
    on load and store, column and transposing passes of 2D/3D transforms, workgroups of 1024
    threads), planar on one side or both, in place, strided, and with different offsets of the
    real and the imaginary array."""
    lib, be = gpu
    K = B
    CP, CI, HP = K.COMPLEX_PLANAR, K.COMPLEX_INTERLEAVED, K.HERMITIAN_PLANAR
    st, text, _ = lib.describe(K.NOTINPLACE, K.COMPLEX_FORWARD, K.SINGLE, [1000], 8,
                               B.PlanDescription(lib).set_data_layout(CP, CP))
    assert st == 0 and "lean planar_in planar_out" in text and " fast" in text, text
    for n in (6, 30, 100, 168, 243, 350, 1000, 1836, 3000, 4096, 7072, 10000):
        H.check(lib, be, K.COMPLEX_FORWARD, [n], 5, K.SINGLE, in_type=CP, out_type=CP)
        H.check(lib, be, K.COMPLEX_INVERSE, [n], 3, K.DOUBLE, in_type=CP, out_type=CP, inplace=True)
        H.check(lib, be, K.COMPLEX_FORWARD, [n], 3, K.DOUBLE, in_type=CP, out_type=CI, scale=0.5)
        H.check(lib, be, K.COMPLEX_INVERSE, [n], 3, K.SINGLE, in_type=CI, out_type=CP)
        H.check(lib, be, K.COMPLEX_FORWARD, [n], 3, K.SINGLE, in_type=CP, out_type=CP, in_offsets=[3, 1],
                out_offsets=[0, 5], in_strides=[2], in_dist=2 * n + 3, out_strides=[3], out_dist=3 * n)
        # even-length real transforms: the half-length kernel with the Hermitian side planar
        H.check(lib, be, K.REAL_FORWARD, [2 * n], 3, K.SINGLE, out_type=HP)
        H.check(lib, be, K.REAL_INVERSE, [2 * n], 3, K.DOUBLE, in_type=HP)
        H.check(lib, be, K.REAL_FORWARD, [2 * n], 3, K.DOUBLE, out_type=HP, out_offsets=[1, 2])
        H.check(lib, be, K.REAL_INVERSE, [2 * n], 3, K.SINGLE, in_type=HP, in_offsets=[2, 1])
    # odd-length real transforms, Bluestein lengths (one kernel and three kernels)
    for n in (9, 77, 625, 1001, 4095, 173, 1009, 2849, 10007):
        H.check(lib, be, K.REAL_FORWARD, [n], 3, K.SINGLE, out_type=HP)
        H.check(lib, be, K.REAL_INVERSE, [n], 3, K.DOUBLE, in_type=HP)
        H.check(lib, be, K.COMPLEX_FORWARD, [n], 3, K.DOUBLE, in_type=CP, out_type=CP)
        H.check(lib, be, K.COMPLEX_INVERSE, [n], 3, K.SINGLE, in_type=CP, out_type=CP, inplace=True)
    for lengths in ([100, 100], [7, 340], [91, 175], [1000, 12], [12, 1000], [360, 360], [541, 24], [64, 64],
                    [25, 17, 135], [44, 68, 20], [9, 10, 6], [100, 77, 16], [173, 14, 27]):
        for prec in (K.SINGLE, K.DOUBLE):
            H.check(lib, be, K.COMPLEX_FORWARD, lengths, 2, prec, in_type=CP, out_type=CP)
            H.check(lib, be, K.COMPLEX_INVERSE, lengths, 2, prec, in_type=CP, out_type=CP, inplace=True)
            H.check(lib, be, K.REAL_FORWARD, lengths, 2, prec, out_type=HP)
            H.check(lib, be, K.REAL_INVERSE, lengths, 2, prec, in_type=HP)


def test_short_rows_with_a_batch_fold_into_full_tiles(gpu):
    """Column passes over rows of a few elements take (column, batch item) pairs as tile entries,
    so that small multi-dimensional transforms in a large batch fill their workgroups: all four
    transform types, in place, padded batch distance, planar, a scale factor, both precisions,
    batches that do not fill the last tile."""
    lib, be = gpu
    K = B
    st, text, _ = lib.describe(K.NOTINPLACE, K.REAL_FORWARD, K.DOUBLE, [4, 5], 1000)
    assert st == 0 and "folded(3)" in text, text
    for lengths, batch in (([4, 5], 1000), ([4, 5], 37), ([6, 10], 333), ([3, 3], 4097), ([5, 7, 3], 211), ([4, 5, 6], 100),
                           ([12, 9], 65), ([2, 2, 2], 1001), ([20, 6], 50), ([33, 5], 77)):
        for prec in (K.SINGLE, K.DOUBLE):
            H.check(lib, be, K.COMPLEX_FORWARD, lengths, batch, prec)
            H.check(lib, be, K.COMPLEX_INVERSE, lengths, batch, prec, inplace=True, scale=0.5)
            H.check(lib, be, K.REAL_FORWARD, lengths, batch, prec)
            H.check(lib, be, K.REAL_INVERSE, lengths, batch, prec)
            H.check(lib, be, K.REAL_FORWARD, lengths, batch, prec, inplace=True)
            H.check(lib, be, K.REAL_INVERSE, lengths, batch, prec, inplace=True)
        total = int(np.prod(lengths))
        strides = [1]
        for v in lengths[:-1]:
            strides.append(strides[-1] * v)
        H.check(lib, be, K.COMPLEX_FORWARD, lengths, batch, K.SINGLE, in_strides=strides, in_dist=total + 3,
                out_strides=strides, out_dist=total + 5)
        H.check(lib, be, K.COMPLEX_FORWARD, lengths, batch, K.DOUBLE, in_type=K.COMPLEX_PLANAR,
                out_type=K.COMPLEX_PLANAR)
        H.check(lib, be, K.REAL_FORWARD, lengths, batch, K.SINGLE, out_type=K.HERMITIAN_PLANAR)


def test_real_rows_of_two_samples(gpu):
    """Real transforms with two samples in the first dimension: the pre/post-processing pass alone
    along that dimension, all layouts."""
    lib, be = gpu
    K = B
    for lengths, batch in (([2], 1000), ([2, 64], 50), ([2, 91, 135], 3), ([2, 7], 4001)):
        for prec in (K.SINGLE, K.DOUBLE):
            H.check(lib, be, K.REAL_FORWARD, lengths, batch, prec)
            H.check(lib, be, K.REAL_INVERSE, lengths, batch, prec)
            H.check(lib, be, K.REAL_FORWARD, lengths, batch, prec, inplace=True, scale=0.5)
            H.check(lib, be, K.REAL_INVERSE, lengths, batch, prec, inplace=True, scale=0.25)
        H.check(lib, be, K.REAL_FORWARD, lengths, batch, K.DOUBLE, out_type=K.HERMITIAN_PLANAR)
        H.check(lib, be, K.REAL_INVERSE, lengths, batch, K.SINGLE, in_type=K.HERMITIAN_PLANAR, scale=2.0)


def test_in_place_real_inverse_without_a_compiled_half_length(gpu):
    """In place, with the standard padded rows, a real inverse transform whose half length has no
    compiled kernel in that precision runs the pre-processing step in place and then the same
    passes as out of place (it used to run one run-time-schedule kernel)."""
    lib, be = gpu
    st, text, _ = lib.describe(B.INPLACE, B.REAL_INVERSE, B.DOUBLE, [11200], 8)
    assert st == 0 and "real pre-process" in text and "split" in text, text
    for n in (11200, 9000, 10000):
        H.check(lib, be, B.REAL_INVERSE, [n], 5, B.DOUBLE, inplace=True)
        H.check(lib, be, B.REAL_INVERSE, [n], 3, B.DOUBLE, inplace=True, scale=0.5)
        H.check(lib, be, B.REAL_FORWARD, [n], 3, B.DOUBLE, inplace=True)
    H.check(lib, be, B.REAL_INVERSE, [11200, 6], 2, B.DOUBLE, inplace=True)


def test_column_tiles_that_span_more_than_two_gib(gpu):
    """A column pass whose tile reaches from the first to the last byte of a 2 GiB array: element
    offsets inside the tile need 29 bits in single precision (129 x 2^21 elements), byte offsets 32."""
    lib, be = gpu
    torch = be.torch
    n, cols = 128, 1 << 21
    st, text, _ = lib.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [n], cols,
                               B.PlanDescription(lib).set_data_layout(B.COMPLEX_INTERLEAVED, B.COMPLEX_INTERLEAVED, None,
                                                                      None, [cols], 1, [cols], 1))
    assert st == 0 and " lean" in text and " fast" in text, text
    gen = torch.Generator(device=be.dev)
    gen.manual_seed(5)
    x = torch.view_as_complex(torch.rand((n, cols, 2), dtype=torch.float32, device=be.dev, generator=gen) - 0.5)
    y = torch.zeros_like(x)
    d = B.PlanDescription(lib).set_data_layout(B.COMPLEX_INTERLEAVED, B.COMPLEX_INTERLEAVED, None, None, [cols], 1,
                                               [cols], 1)
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [n], cols, d, lib=lib)
    plan.execute([x.data_ptr()], [y.data_ptr()])
    torch.cuda.synchronize()
    # the checker on three groups of columns: the first, the last and some in the middle
    for lo in (0, cols // 2 - 77, cols - 256):
        xs = x[:, lo:lo + 256].cpu().numpy().astype(np.complex128)
        ref = orc.transform(B.COMPLEX_FORWARD, [n], 256, np.ascontiguousarray(xs.T), ld=False).reshape(256, n).T
        l2, linf = orc.rel_norms(y[:, lo:lo + 256].cpu().numpy().astype(np.complex128).reshape(-1), ref.reshape(-1))
        assert l2 <= 1e-5 and linf <= 1e-5, (lo, l2, linf)
    # every column was written
    assert int((y == 0).sum()) == 0
    plan.destroy()


@pytest.mark.parametrize("n", [16384, 32768, 65536, 2 ** 18, 2 ** 20, 6000, 30030, 10007, 4099, 8198, 65537])
def test_long_1d(gpu, n):
    lib, be = gpu
    H.check(lib, be, B.COMPLEX_FORWARD, [n], 3, B.SINGLE)
    H.check(lib, be, B.COMPLEX_INVERSE, [n], 2, B.DOUBLE, inplace=True)
    if n % 2 == 0:
        H.check(lib, be, B.REAL_FORWARD, [n], 3, B.DOUBLE)
        H.check(lib, be, B.REAL_INVERSE, [n], 3, B.SINGLE)
        H.check(lib, be, B.REAL_FORWARD, [n], 2, B.SINGLE, inplace=True)
        H.check(lib, be, B.REAL_INVERSE, [n], 2, B.DOUBLE, inplace=True)


def test_four_pass_split(gpu, monkeypatch):
    """one more strided pass than the longest lengths of three passes need, asked for at lengths
    the checker finishes (the lengths that need it are run by tests/test_reference_matrix.py)"""
    lib, be = gpu
    monkeypatch.setenv("ROCFFT_AMD_SPLIT_LEVELS", "4")
    for n in (65536, 2 ** 20, 3 ** 9, 5 ** 8, 30030):
        H.check(lib, be, B.COMPLEX_FORWARD, [n], 2, B.SINGLE)
        H.check(lib, be, B.COMPLEX_INVERSE, [n], 1, B.DOUBLE, inplace=True, scale=0.5)
    monkeypatch.setenv("ROCFFT_AMD_SPLIT_LEVELS", "3")
    H.check(lib, be, B.COMPLEX_FORWARD, [32768], 2, B.SINGLE)
    H.check(lib, be, B.COMPLEX_FORWARD, [2 ** 17], 2, B.DOUBLE)


def test_three_level_chirp_z(gpu, monkeypatch):
    """the chirp-z form for convolution lengths beyond 2^26, asked for at lengths the checker
    finishes (tests/test_reference_matrix.py runs a prime that needs it)"""
    lib, be = gpu
    monkeypatch.setenv("ROCFFT_AMD_BLU3", "64,128")
    for n in (100003, 1000003):  # 2^18 = 32 x 64 x 128, 2^21 = 256 x 64 x 128
        H.check(lib, be, B.COMPLEX_FORWARD, [n], 2, B.SINGLE)
        H.check(lib, be, B.COMPLEX_INVERSE, [n], 1, B.DOUBLE, inplace=True, scale=0.5)
    monkeypatch.setenv("ROCFFT_AMD_BLU3", "16,4096")
    H.check(lib, be, B.COMPLEX_FORWARD, [1000003], 3, B.DOUBLE)
    H.check(lib, be, B.COMPLEX_FORWARD, [7, 100003], 1, B.SINGLE)
    H.check(lib, be, B.COMPLEX_FORWARD, [100003, 3], 1, B.SINGLE)


@pytest.mark.parametrize("lengths", [[8193], [10007], [19683], [15625], [100003], [9999, 3], [3, 9999]])
def test_long_odd_real(gpu, lengths):
    lib, be = gpu
    H.check(lib, be, B.REAL_FORWARD, lengths, 2, B.DOUBLE)
    H.check(lib, be, B.REAL_INVERSE, lengths, 2, B.SINGLE)
    H.check(lib, be, B.REAL_FORWARD, lengths, 2, B.SINGLE, inplace=True, scale=0.25)
    H.check(lib, be, B.REAL_INVERSE, lengths, 2, B.DOUBLE, inplace=True)


@pytest.mark.parametrize("lengths", [[9, 2053], [64, 2053], [11, 2947], [40, 4099], [1155, 2084], [3, 5, 2311],
                                     [6, 20011]])
def test_bluestein_in_a_strided_dimension(gpu, lengths):
    """A chirp-z dimension whose padded length needs the three-kernel form, behind a contiguous
    dimension: the padded signals keep the columns innermost; the signal is shorter than the
    row factor of the padded length in the first cases (loads of the padding must stay inside
    the array)."""
    lib, be = gpu
    H.check(lib, be, B.COMPLEX_FORWARD, lengths, 2, B.SINGLE)
    H.check(lib, be, B.COMPLEX_INVERSE, lengths, 1, B.DOUBLE, inplace=True)
    H.check(lib, be, B.REAL_FORWARD, lengths, 2, B.DOUBLE)
    H.check(lib, be, B.REAL_INVERSE, lengths, 1, B.SINGLE)


@pytest.mark.parametrize("lengths", [[8, 8], [64, 64], [100, 30], [17, 19], [1024, 1024], [4096, 64], [64, 4096],
                                     [8, 8, 8], [16, 8, 4], [30, 20, 10], [128, 32, 8], [5, 7, 9], [8192, 4], [4, 8192], [64, 64, 64],
                                     [128, 128, 128], [512, 16, 16], [16, 512, 4], [8, 4, 512], [1, 8], [8, 1, 4]])
def test_multi_dim(gpu, lengths):
    lib, be = gpu
    for kind in range(4):
        H.check(lib, be, kind, lengths, 2, B.DOUBLE)
        H.check(lib, be, kind, lengths, 1, B.SINGLE, inplace=True)


def test_small_2d_in_one_workgroup(gpu):
    """8..64 x 8..64 complex transforms run as one kernel; also as the first two dimensions of a
    3D transform, in place, with a scale factor, and with fewer transforms than a workgroup takes."""
    lib, be = gpu
    for a in (8, 16, 32, 64):
        for b_ in (8, 16, 32, 64):
            print("2d", a, b_, flush=True)
            H.check(lib, be, B.COMPLEX_FORWARD, [a, b_], 37, B.SINGLE)
            H.check(lib, be, B.COMPLEX_INVERSE, [a, b_], 5, B.DOUBLE, inplace=True, scale=0.5)
            H.check(lib, be, B.COMPLEX_FORWARD, [a, b_, 6], 3, B.DOUBLE)
            H.check(lib, be, B.COMPLEX_INVERSE, [a, b_], 1, B.SINGLE)
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [16, 16], 100, lib=lib)
    assert [name for name, _ in plan.passes()] == ["2D fft 16x16 in one workgroup"]
    # a layout the one-kernel path does not take (padded rows) still works, in two passes
    H.check(lib, be, B.COMPLEX_FORWARD, [16, 16], 4, B.SINGLE, in_strides=[1, 20], in_dist=400)


def test_small_real_2d_in_one_workgroup(gpu):
    """8..64 x 8..64 real transforms, both directions, run as one kernel (half-length rows, fused
    pre/post-processing on the LDS tile, columns of the N/2+1 bins); also in place (padded rows),
    as the first two dimensions of a 3D transform, and with a scale factor."""
    lib, be = gpu
    for a in (8, 16, 32, 64):
        for b_ in (8, 16, 32, 64):
            print("real 2d", a, b_, flush=True)
            H.check(lib, be, B.REAL_FORWARD, [a, b_], 37, B.SINGLE)
            H.check(lib, be, B.REAL_INVERSE, [a, b_], 37, B.DOUBLE)
            H.check(lib, be, B.REAL_FORWARD, [a, b_], 5, B.DOUBLE, inplace=True, scale=0.5)
            H.check(lib, be, B.REAL_INVERSE, [a, b_], 5, B.SINGLE, inplace=True, scale=0.25)
            H.check(lib, be, B.REAL_FORWARD, [a, b_, 6], 3, B.SINGLE)
            H.check(lib, be, B.REAL_INVERSE, [a, b_, 6], 3, B.DOUBLE)
    plan = B.Plan(B.NOTINPLACE, B.REAL_INVERSE, B.SINGLE, [16, 16, 16], 10, lib=lib)
    assert [name for name, _ in plan.passes()] == ["column fft n=16", "2D real inverse fft 16x16 in one workgroup"]
    # an out-of-place 2D real inverse through the one-kernel path leaves its input alone
    import torch
    x = torch.view_as_complex(torch.rand((9, 32, 17, 2), device=be.dev) - 0.5).contiguous()
    keep = x.clone()
    y = torch.empty((9, 32, 32), device=be.dev)
    plan = B.Plan(B.NOTINPLACE, B.REAL_INVERSE, B.SINGLE, [32, 32], 9, lib=lib)
    plan.execute([x.data_ptr()], [y.data_ptr()])
    torch.cuda.synchronize()
    assert torch.equal(x, keep)


def test_large_square_2d(gpu):
    # both dimensions beyond the longest single-kernel length
    lib, be = gpu
    H.check(lib, be, B.COMPLEX_FORWARD, [8192, 8192], 1, B.SINGLE)
    H.check(lib, be, B.COMPLEX_INVERSE, [4096, 2048], 2, B.DOUBLE, inplace=True)


def test_layouts(gpu):
    lib, be = gpu
    K = B
    H.check(lib, be, K.COMPLEX_FORWARD, [64], 3, K.DOUBLE, in_strides=[3], in_dist=200, out_strides=[2],
            out_dist=130, in_offsets=[5, 0], out_offsets=[7, 0])
    H.check(lib, be, K.COMPLEX_FORWARD, [128], 8, K.SINGLE, in_strides=[8], in_dist=1, out_strides=[8],
            out_dist=1)
    H.check(lib, be, K.COMPLEX_INVERSE, [30, 4], 2, K.DOUBLE, in_type=K.COMPLEX_PLANAR,
            out_type=K.COMPLEX_PLANAR, in_offsets=[3, 9], out_offsets=[2, 1])
    H.check(lib, be, K.COMPLEX_FORWARD, [16384], 2, K.SINGLE, in_type=K.COMPLEX_INTERLEAVED,
            out_type=K.COMPLEX_PLANAR)
    H.check(lib, be, K.REAL_FORWARD, [32, 6], 2, K.DOUBLE, out_type=K.HERMITIAN_PLANAR)
    H.check(lib, be, K.REAL_INVERSE, [32, 6], 2, K.DOUBLE, in_type=K.HERMITIAN_PLANAR)
    H.check(lib, be, K.REAL_FORWARD, [20, 6], 2, K.SINGLE, in_strides=[1, 23], in_dist=150,
            out_strides=[1, 13], out_dist=90)
    H.check(lib, be, K.REAL_INVERSE, [21, 6], 2, K.SINGLE, in_strides=[2, 30], in_dist=200,
            out_strides=[1, 25], out_dist=160)
    H.check(lib, be, K.COMPLEX_FORWARD, [16, 8], 2, K.DOUBLE, out_strides=[8, 1], out_dist=128)
    for kind, lengths in [(0, [64]), (1, [16384]), (2, [64]), (2, [16384]), (3, [64]), (3, [16384]), (0, [97]),
                          (0, [4099]), (0, [8, 8, 8]), (2, [8, 8]), (3, [7, 8])]:
        H.check(lib, be, kind, lengths, 2, K.DOUBLE, scale=1.0 / 64)


def test_no_stray_writes(gpu):
    lib, be = gpu
    for kind, lengths, kw in [(0, [64], dict(out_strides=[3], out_dist=250)),
                              (0, [16384], dict(out_strides=[2], out_dist=40000)),
                              (2, [30, 4], dict(out_strides=[2, 40], out_dist=200)),
                              (3, [32, 4], dict(out_strides=[1, 37], out_dist=170)),
                              (0, [97], dict(out_strides=[2], out_dist=300))]:
        y, x, touched = H.run_transform(lib, be, kind, lengths, 2, B.SINGLE, return_buffers=True, **kw)
        for raw, mask in touched:
            assert np.all(raw[~mask[:raw.size]] == H.GUARD), (kind, lengths)
        assert orc.rel_norms(y, H.reference(kind, lengths, 2, x, B.SINGLE))[0] < 1e-5


def test_c2r_ignores_imaginary_dc_and_nyquist(gpu):
    lib, be = gpu
    for n in (8, 8192, 65536, 9):
        h = H.make_input(B.REAL_INVERSE, [n], 1)
        h2 = h.copy()
        h2[0, 0] += 2.5j
        if n % 2 == 0:
            h2[0, -1] -= 1.5j
        y1, _ = H.run_transform(lib, be, B.REAL_INVERSE, [n], 1, B.DOUBLE, x=h)
        y2, _ = H.run_transform(lib, be, B.REAL_INVERSE, [n], 1, B.DOUBLE, x=h2)
        assert np.array_equal(y1, y2), n


def test_streaming_one_workgroup_kernel_batches_and_layouts(gpu):
    """The one-workgroup 32768-point kernel walks through the transforms of a launch, a workgroup
    taking every G-th one and prefetching its next: batch counts below, at and above the
    number of workgroups (1024 on MI355X), rows that alternate between 16- and 8-byte alignment
    (32769 bins), padded distances, a second dimension, scaling, both complex directions."""
    lib, be = gpu
    torch = be.torch
    # against the checker: few transforms, every mode, odd row alignments
    for kind, lengths, batch, kw in [
            (B.REAL_FORWARD, [65536], 1, {}), (B.REAL_INVERSE, [65536], 1, {}),
            (B.REAL_FORWARD, [65536], 5, {"scale": 0.5}), (B.REAL_INVERSE, [65536], 5, {"scale": 1.0 / 65536}),
            (B.COMPLEX_FORWARD, [32768], 3, {}), (B.COMPLEX_INVERSE, [32768], 3, {"scale": 2.0}),
            (B.COMPLEX_FORWARD, [32768], 2, {"inplace": True}),
            (B.REAL_FORWARD, [65536], 3, {"in_strides": [1], "in_dist": 65536 + 12, "out_strides": [1], "out_dist": 32769 + 3}),
            (B.REAL_INVERSE, [65536], 3, {"in_strides": [1], "in_dist": 32769 + 2, "out_strides": [1], "out_dist": 65536 + 4}),
            (B.REAL_FORWARD, [65536, 3], 2, {}), (B.REAL_INVERSE, [65536, 3], 2, {}), (B.COMPLEX_FORWARD, [32768, 2], 2, {})]:
        H.check(lib, be, kind, lengths, batch, B.SINGLE, **kw)
    # many transforms: round trip and a cross-check of a few rows against torch.fft
    n = 65536
    for batch in (255, 1023, 1024, 1025, 2500):
        x = (inputs.torch_uniform01(torch, be.dev, 40 + batch, 0, n * batch) * 2 - 1).to(torch.float32).reshape(batch, n)
        h = torch.full((batch, n // 2 + 1), float("nan"), dtype=torch.complex64, device=be.dev)
        y = torch.full((batch, n), float("nan"), dtype=torch.float32, device=be.dev)
        fwd = B.Plan(B.NOTINPLACE, B.REAL_FORWARD, B.SINGLE, [n], batch, lib=lib)
        inv = B.Plan(B.NOTINPLACE, B.REAL_INVERSE, B.SINGLE, [n], batch, lib=lib)
        fwd.execute([x.data_ptr()], [h.data_ptr()])
        inv.execute([h.data_ptr()], [y.data_ptr()])
        torch.cuda.synchronize()
        rows = sorted(set([0, 1, batch // 2, batch - 2, batch - 1]))
        ref = torch.fft.rfft(x[rows].double(), dim=1)
        l2, li = tnorm(torch, h[rows], ref)
        assert l2 <= 1e-5 and li <= 1e-5, (batch, l2, li)
        l2, li = tnorm(torch, y / n, x)
        assert l2 <= 1e-5 and li <= 1e-5, (batch, l2, li)
        # every row, cheaply: Parseval per row
        e_in = (x.double() ** 2).sum(dim=1)
        hh = torch.view_as_real(h).double()
        e_out = (2 * (hh ** 2).sum(dim=(1, 2)) - hh[:, 0, 0] ** 2 - hh[:, -1, 0] ** 2) / n
        assert ((e_out / e_in - 1).abs().max().item()) < 1e-5, batch


def test_buffers_aligned_to_a_scalar_only(gpu):
    """Base pointers offset by one scalar.  The kernels that move (re, im) pairs with one
    access have no form for such buffers; plans that use them carry a second pass list made
    of the tile kernel alone, which the executor takes.  The reference accepts such buffers
    (its kernels address scalars)."""
    lib, be = gpu
    torch = be.torch
    cases = [(B.REAL_FORWARD, B.SINGLE, [65536], 3), (B.REAL_INVERSE, B.SINGLE, [65536], 3),
             (B.COMPLEX_FORWARD, B.SINGLE, [32768], 2), (B.COMPLEX_FORWARD, B.SINGLE, [16384], 3),
             (B.COMPLEX_INVERSE, B.SINGLE, [32, 32], 5), (B.REAL_FORWARD, B.SINGLE, [16, 16], 7),
             (B.COMPLEX_FORWARD, B.DOUBLE, [64, 16], 3)]
    for kind, prec, lengths, batch in cases:
        rt = torch.float32 if prec == B.SINGLE else torch.float64
        total = int(np.prod(lengths))
        herm = total // lengths[0] * (lengths[0] // 2 + 1)
        n_in = {B.REAL_FORWARD: total, B.REAL_INVERSE: 2 * herm}.get(kind, 2 * total) * batch
        n_out = {B.REAL_FORWARD: 2 * herm, B.REAL_INVERSE: total}.get(kind, 2 * total) * batch
        plan = B.Plan(B.NOTINPLACE, kind, prec, lengths, batch, lib=lib)
        x = (inputs.torch_uniform01(torch, be.dev, 31, 0, n_in) - 0.5).to(rt)
        if kind == B.REAL_INVERSE:
            # a Hermitian input: the forward transform of real data
            fwd = B.Plan(B.NOTINPLACE, B.REAL_FORWARD, prec, lengths, batch, lib=lib)
            real = (inputs.torch_uniform01(torch, be.dev, 32, 0, total * batch) - 0.5).to(rt)
            fwd.execute([real.data_ptr()], [x.data_ptr()])
            torch.cuda.synchronize()
        want = torch.full((n_out,), float("nan"), dtype=rt, device=be.dev)
        plan.execute([x.clone().data_ptr()], [want.data_ptr()])
        torch.cuda.synchronize()
        # the same data one scalar into larger allocations
        xin = torch.zeros(n_in + 1, dtype=rt, device=be.dev)
        xin[1:] = x
        yout = torch.full((n_out + 2,), 7.0, dtype=rt, device=be.dev)
        info = B.ExecutionInfo(lib)
        wb = plan.work_buffer_size
        if wb:
            work = torch.empty(wb, dtype=torch.uint8, device=be.dev)
            info.set_work_buffer(work.data_ptr(), wb)
        plan.execute([xin[1:].data_ptr()], [yout[1:].data_ptr()], info)
        torch.cuda.synchronize()
        assert yout[0].item() == 7.0 and yout[-1].item() == 7.0, (kind, lengths)
        got = yout[1:-1]
        assert torch.isfinite(got).all(), (kind, lengths)
        l2, li = tnorm(torch, got, want)
        tol = 1e-5 if prec == B.SINGLE else 1e-13
        assert l2 <= tol and li <= tol, (kind, lengths, l2, li)
        # and without a caller's work buffer (the library allocates what this pass list needs)
        yout.fill_(7.0)
        plan.execute([xin[1:].data_ptr()], [yout[1:].data_ptr()])
        torch.cuda.synchronize()
        l2, li = tnorm(torch, yout[1:-1], want)
        assert l2 <= tol and li <= tol, (kind, lengths, l2, li)


def test_work_buffer_contract(gpu):
    lib, be = gpu
    torch = be.torch
    n = 8191  # double precision: three Bluestein kernels and a work buffer
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.DOUBLE, [n], 1, lib=lib)
    need = plan.work_buffer_size
    assert need > 0
    x = torch.zeros(n, dtype=torch.complex128, device=be.dev)
    x[1] = 1
    y = torch.zeros_like(x)
    plan.execute([x.data_ptr()], [y.data_ptr()])  # scratch allocated by execute
    torch.cuda.synchronize()
    want = np.exp(-2j * np.pi * np.arange(n) / n)
    assert np.allclose(y.cpu().numpy(), want, atol=1e-4)
    info = B.ExecutionInfo(lib)
    small = torch.zeros(need // 2, dtype=torch.uint8, device=be.dev)
    info.set_work_buffer(small.data_ptr(), need // 2)
    assert plan.execute_status([x.data_ptr()], [y.data_ptr()], info) == B.STATUS_INVALID_WORK_BUFFER


def test_streams_threads_and_graph_capture(gpu):
    lib, be = gpu
    torch = be.torch
    n, batch = 4096, 64
    x = inputs.torch_uniform01(torch, be.dev, 5, 0, 2 * n * batch).to(torch.float32) - 0.5
    x = torch.view_as_complex(x.reshape(batch, n, 2).contiguous())
    ref = torch.fft.fft(x, dim=1)
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [n], batch, lib=lib)
    # several user streams (reference clients/tests/multithread_test.cpp:310-348)
    outs, streams = [], [torch.cuda.Stream() for _ in range(3)]
    torch.cuda.synchronize()
    for s in streams:
        y = torch.empty_like(x)
        info = B.ExecutionInfo(lib).set_stream(s.cuda_stream)
        plan.execute([x.data_ptr()], [y.data_ptr()], info)
        outs.append(y)
    torch.cuda.synchronize()
    for y in outs:
        assert tnorm(torch, y, ref)[0] < 1e-5
    # plan creation and execution from several host threads (multithread_test.cpp:255-278)
    errs = []

    def worker(k):
        try:
            p = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [n >> k], batch << k, lib=lib)
            s = torch.cuda.Stream()
            y = torch.empty_like(x)
            p.execute([x.data_ptr()], [y.data_ptr()], B.ExecutionInfo(lib).set_stream(s.cuda_stream))
            s.synchronize()
            want = torch.fft.fft(x.reshape(batch << k, n >> k), dim=1)
            if tnorm(torch, y.reshape(batch << k, n >> k), want)[0] > 1e-5:
                errs.append(k)
        except Exception as e:  # noqa: BLE001
            errs.append(repr(e))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(4)]
    [t.start() for t in threads]
    [t.join() for t in threads]
    assert not errs, errs
    # rocfft_execute can be captured into a graph and replayed (clients/tests/hipGraph_test.cpp:272)
    y = torch.zeros_like(x)
    xin = x.clone()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            info = B.ExecutionInfo(lib).set_stream(torch.cuda.current_stream().cuda_stream)
            plan.execute([xin.data_ptr()], [y.data_ptr()], info)
    torch.cuda.synchronize()
    for rep in range(3):
        xin.copy_(x * (rep + 1))
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert tnorm(torch, y, ref * (rep + 1))[0] < 1e-5, rep


# ------------------------------------------------------------------ the five configurations, full size
def golden_check(cfg_id, y_rows):
    g = np.load(os.path.join(GOLDEN, "cfg%d.npz" % cfg_id))
    rows = int(g["rows"])
    y = y_rows[:rows]
    scale = g["l2"][:rows, None] / np.sqrt(y.shape[1])
    tol = H.tolerance(B.SINGLE if inputs.CONFIGS[cfg_id]["precision"] == "single" else B.DOUBLE)
    err = np.max(np.abs(y[:, g["bins"]] - g["values"][:rows]) / scale)
    assert err < 10 * tol, err  # a single bin against the rms bin magnitude
    assert np.max(np.abs(np.sqrt((np.abs(y) ** 2).sum(axis=1)) / g["l2"][:rows] - 1)) < tol


def run_plan(lib, torch, plan, src, dst):
    info = B.ExecutionInfo(lib)
    wb = plan.work_buffer_size
    work = None
    if wb:
        work = torch.empty(wb, dtype=torch.uint8, device=src.device)
        info.set_work_buffer(work.data_ptr(), wb)
    plan.execute([src.data_ptr()], None if dst is None else [dst.data_ptr()], info)
    torch.cuda.synchronize()


def test_config1_c2c_4096_inplace(gpu):
    lib, be = gpu
    torch = be.torch
    x = inputs.torch_config_input(torch, be.dev, 1)
    buf = x.clone()
    plan = B.Plan(B.INPLACE, B.COMPLEX_FORWARD, B.SINGLE, [4096], 1024, lib=lib)
    run_plan(lib, torch, plan, buf, None)
    y = buf.cpu().numpy().astype(np.complex128)
    ref = orc.transform(orc.COMPLEX_FORWARD, [4096], 1024, x.cpu().numpy().astype(np.complex128))
    l2, li = orc.rel_norms(y.reshape(-1), ref)
    assert l2 <= 1e-5 and li <= 1e-5, (l2, li)
    golden_check(1, y)
    assert tnorm(torch, buf, torch.fft.fft(x, dim=1))[0] <= 1e-5  # reference rocFFT via hipFFT


def test_config2_r2c_c2r_65536(gpu):
    lib, be = gpu
    torch = be.torch
    n, batch = 65536, 4096
    x = inputs.torch_config_input(torch, be.dev, 2)
    keep = x.clone()
    h = torch.empty((batch, n // 2 + 1), dtype=torch.complex64, device=be.dev)
    fwd = B.Plan(B.NOTINPLACE, B.REAL_FORWARD, B.SINGLE, [n], batch, lib=lib)
    run_plan(lib, torch, fwd, x, h)
    assert torch.equal(x, keep)  # out-of-place forward keeps its input
    head = h[:8].cpu().numpy().astype(np.complex128)
    ref = orc.transform(orc.REAL_FORWARD, [n], 8, x[:8].cpu().numpy().astype(np.float64)).reshape(8, -1)
    l2, li = orc.rel_norms(head, ref)
    assert l2 <= 1e-5 and li <= 1e-5, (l2, li)
    golden_check(2, head)
    assert tnorm(torch, h, torch.fft.rfft(x, dim=1))[0] <= 1e-5
    assert h[:, 0].imag.abs().max().item() == 0 and h[:, -1].imag.abs().max().item() == 0
    # Parseval over the whole batch: sum |x|^2 * n = |X0|^2 + |Xnyq|^2 + 2 sum_{0<k<n/2} |Xk|^2
    e_in = (x.double() ** 2).sum().item() * n
    hh = h.abs().double() ** 2
    e_out = (2 * hh.sum() - hh[:, 0].sum() - hh[:, -1].sum()).item()
    assert abs(e_out / e_in - 1) < 1e-5
    # unnormalised round trip (reference shared/accuracy_test.h:685-861)
    back = torch.empty_like(x)
    inv = B.Plan(B.NOTINPLACE, B.REAL_INVERSE, B.SINGLE, [n], batch, lib=lib)
    run_plan(lib, torch, inv, h, back)
    l2, li = tnorm(torch, back / n, x)
    assert l2 <= 1e-5 and li <= 1e-5, (l2, li)


def test_config3_c2c_4096x4096(gpu):
    lib, be = gpu
    torch = be.torch
    x = inputs.torch_config_input(torch, be.dev, 3)
    keep = x.clone()
    y = torch.empty_like(x)
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [4096, 4096], 8, lib=lib)
    run_plan(lib, torch, plan, x, y)
    assert torch.equal(x, keep)
    golden_check(3, y[:1].cpu().numpy().astype(np.complex128))
    ref = torch.fft.fft2(x.reshape(8, 4096, 4096)).reshape(8, -1)
    l2, li = tnorm(torch, y, ref)
    assert l2 <= 1e-5 and li <= 1e-5, (l2, li)
    del ref
    # spot bins of the last batch entry from the 2D DFT definition (separable: rows then one column sum)
    xb = x[7].reshape(4096, 4096).cpu().numpy().astype(np.complex128)
    for (k1, k0) in [(0, 0), (1, 4095), (2049, 77)]:
        col = (xb * np.exp(-2j * np.pi * k0 * np.arange(4096) / 4096)[None, :]).sum(axis=1)
        want = orc.dft_bin(col, k1)
        got = complex(y[7, k1 * 4096 + k0].item())
        assert abs(got - want) / 4096 < 1e-4
    # round trip
    back = torch.empty_like(x)
    inv = B.Plan(B.NOTINPLACE, B.COMPLEX_INVERSE, B.SINGLE, [4096, 4096], 8, lib=lib)
    run_plan(lib, torch, inv, y, back)
    l2, li = tnorm(torch, back / (4096.0 * 4096.0), x)
    assert l2 <= 1e-5 and li <= 1e-5, (l2, li)


def test_config4_r2c_c2r_512cubed_double(gpu):
    lib, be = gpu
    torch = be.torch
    n = 512
    x = inputs.torch_config_input(torch, be.dev, 4)
    keep = x.clone()
    h = torch.empty((1, n * n * (n // 2 + 1)), dtype=torch.complex128, device=be.dev)
    fwd = B.Plan(B.NOTINPLACE, B.REAL_FORWARD, B.DOUBLE, [n, n, n], 1, lib=lib)
    run_plan(lib, torch, fwd, x, h)
    assert torch.equal(x, keep)
    golden_check(4, h.cpu().numpy())
    ref = torch.fft.rfftn(x.reshape(n, n, n)).reshape(1, -1)
    l2, li = tnorm(torch, h, ref)
    assert l2 <= 1e-13 and li <= 1e-13, (l2, li)
    del ref
    back = torch.empty_like(x)
    inv = B.Plan(B.NOTINPLACE, B.REAL_INVERSE, B.DOUBLE, [n, n, n], 1, lib=lib)
    run_plan(lib, torch, inv, h.clone(), back)  # the inverse may overwrite its input
    l2, li = tnorm(torch, back / float(n ** 3), x)
    assert l2 <= 1e-13 and li <= 1e-13, (l2, li)


def test_config5_bluestein_prime_1000003_double(gpu):
    lib, be = gpu
    torch = be.torch
    n, batch = 1000003, 16
    x = inputs.torch_config_input(torch, be.dev, 5)
    keep = x.clone()
    y = torch.empty_like(x)
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.DOUBLE, [n], batch, lib=lib)
    run_plan(lib, torch, plan, x, y)
    assert torch.equal(x, keep)
    yh = y.cpu().numpy()
    golden_check(5, yh)
    # full comparison of two rows with the long double checker, spot bins on the others
    xh = x.cpu().numpy()
    ref = orc.fft1d(xh[:2], ld=True)
    l2, li = orc.rel_norms(yh[:2], ref)
    assert l2 <= 1e-13 and li <= 1e-13, (l2, li)
    scale = np.abs(yh).max()
    for b in (2, 9, 15):
        for k in (0, 1, 500001, n - 1):
            assert abs(yh[b, k] - orc.dft_bin(xh[b], k)) / scale < 1e-13
    l2, li = tnorm(torch, y, torch.fft.fft(x, dim=1))
    assert l2 <= 1e-13, (l2, li)  # reference rocFFT; its own error is in this figure too
    back = torch.empty_like(x)
    inv = B.Plan(B.NOTINPLACE, B.COMPLEX_INVERSE, B.DOUBLE, [n], batch, lib=lib)
    run_plan(lib, torch, inv, y, back)
    l2, li = tnorm(torch, back / float(n), x)
    assert l2 <= 1e-13 and li <= 1e-13, (l2, li)
