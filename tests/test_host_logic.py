"""CPU tests of the host side: the C ABI surface, the status-code contract of
the rocfft.h entry points, the planner's pass lists, and -- through the host
emulation of the runtime layer (tests/emu) -- the numerics of every pass kind
the planner can emit, including strides, offsets, planar arrays and scaling.

Status expectations follow the reference (library/src/plan.cpp:73-74, :729-779,
:2968, :3139-3140, :3279-3289; library/src/transform.cpp:58-59, :80-81,
:339-340, :436-442) and its unit tests (clients/tests/unit_test.cpp:59-345).
"""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

import helpers as H
import rocfft_amd.binding as B
from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = H.HostBackend()


# ------------------------------------------------------------------ ABI surface
def declared_functions():
    names = []
    for header in ("include/rocfft/rocfft.h", "include/rocfft_amd.h"):
        text = open(os.path.join(ROOT, header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(rocfft_[a-z_]+)\s*\(", text)
    return sorted(set(names))


def test_product_library_exports_every_declared_symbol():
    path = B.library_path()
    assert os.path.exists(path), "build the library first (__graft_entry__.build())"
    out = subprocess.check_output(["nm", "-D", "--defined-only", path]).decode()
    exported = set(re.findall(r" T (rocfft_\w+)", out))
    declared = declared_functions()
    assert len(declared) == 35  # the 29 entry points of rocfft.h plus the 6 rocfft_amd_* extensions
    assert set(declared) <= exported, set(declared) - exported
    assert set(declared) == set(B.EXPORTED_SYMBOLS)
    # loads without a GPU and answers host-only calls
    lib = B.Library(path)
    assert lib.version().startswith("1.0.")


def test_enum_values_match_reference_header():
    text = open(os.path.join(ROOT, "include/rocfft/rocfft.h")).read()
    for name, val in [("rocfft_status_invalid_work_buffer", 8), ("rocfft_transform_type_real_inverse", 3),
                      ("rocfft_precision_half", 2), ("rocfft_placement_notinplace", 1),
                      ("rocfft_array_type_unset", 5), ("rocfft_array_type_hermitian_planar", 4),
                      ("rocfft_comm_mpi", 1)]:
        assert re.search(r"%s\s*=\s*%d\b" % (name, val), text), name


def test_plan_create_without_gpu_fails_loudly():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = B.Library()
    with pytest.raises(B.RocfftError) as e:
        B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [64], 1, lib=lib)
    assert e.value.status == B.STATUS_FAILURE


# ------------------------------------------------------------------ status codes
def test_status_codes(emu):
    c = emu.c
    ln = (ctypes.c_size_t * 4)(8, 8, 8, 8)
    h = ctypes.c_void_p()
    assert c.rocfft_plan_create(ctypes.byref(h), 1, 0, 0, 4, ln, 1, None) == B.STATUS_INVALID_DIMENSIONS
    assert c.rocfft_plan_create(ctypes.byref(h), 1, 0, 0, 0, ln, 1, None) == B.STATUS_INVALID_DIMENSIONS
    assert c.rocfft_plan_create(ctypes.byref(h), 1, 0, B.HALF, 1, ln, 1, None) == 0
    c.rocfft_plan_destroy(h)
    assert c.rocfft_plan_create(ctypes.byref(h), 1, 0, 7, 1, ln, 1, None) == B.STATUS_FAILURE  # no such precision

    def create(placement, kind, it, ot):
        d = B.PlanDescription(emu).set_data_layout(it, ot)
        return c.rocfft_plan_create(ctypes.byref(h), placement, kind, 0, 1, ln, 1, d.handle)

    bad = B.STATUS_INVALID_ARRAY_TYPE
    assert create(B.NOTINPLACE, B.COMPLEX_FORWARD, B.REAL, B.COMPLEX_INTERLEAVED) == bad
    assert create(B.NOTINPLACE, B.COMPLEX_FORWARD, B.COMPLEX_INTERLEAVED, B.HERMITIAN_INTERLEAVED) == bad
    assert create(B.INPLACE, B.COMPLEX_FORWARD, B.COMPLEX_INTERLEAVED, B.COMPLEX_PLANAR) == bad
    assert create(B.NOTINPLACE, B.REAL_FORWARD, B.COMPLEX_INTERLEAVED, B.HERMITIAN_INTERLEAVED) == bad
    assert create(B.INPLACE, B.REAL_FORWARD, B.REAL, B.HERMITIAN_PLANAR) == bad
    assert create(B.NOTINPLACE, B.REAL_INVERSE, B.HERMITIAN_INTERLEAVED, B.COMPLEX_INTERLEAVED) == bad
    assert create(B.INPLACE, B.REAL_INVERSE, B.HERMITIAN_PLANAR, B.REAL) == bad
    assert create(B.NOTINPLACE, B.COMPLEX_FORWARD, B.COMPLEX_INTERLEAVED, B.COMPLEX_PLANAR) == 0
    c.rocfft_plan_destroy(h)

    d = B.PlanDescription(emu)
    assert c.rocfft_plan_description_set_scale_factor(d.handle, float("nan")) == B.STATUS_INVALID_ARG_VALUE
    assert c.rocfft_plan_description_set_scale_factor(d.handle, float("inf")) == B.STATUS_INVALID_ARG_VALUE
    assert c.rocfft_plan_description_set_scale_factor(d.handle, 0.5) == 0

    info = B.ExecutionInfo(emu)
    assert c.rocfft_execution_info_set_work_buffer(info.handle, None, 16) == B.STATUS_INVALID_WORK_BUFFER
    fn = (ctypes.c_void_p * 1)(1)
    assert c.rocfft_execution_info_set_load_callback(info.handle, fn, None, 8) == B.STATUS_INVALID_ARG_VALUE
    assert c.rocfft_execution_info_set_store_callback(info.handle, fn, None, 8) == B.STATUS_INVALID_ARG_VALUE
    assert c.rocfft_execution_info_set_load_callback(info.handle, fn, None, 0) == 0
    assert c.rocfft_execution_info_set_load_callback(info.handle, None, None, 0) == 0

    assert c.rocfft_execute(None, None, None, None) == B.STATUS_FAILURE
    n = ctypes.c_size_t()
    assert c.rocfft_plan_get_work_buffer_size(None, ctypes.byref(n)) == B.STATUS_FAILURE
    assert c.rocfft_get_version_string(None, 64) == B.STATUS_FAILURE
    small = ctypes.create_string_buffer(2)
    assert c.rocfft_get_version_string(small, 2) == B.STATUS_INVALID_ARG_VALUE
    # destroying null handles is fine
    assert c.rocfft_plan_description_destroy(None) == 0
    assert c.rocfft_execution_info_destroy(None) == 0
    # setup/cleanup may repeat
    assert c.rocfft_setup() == 0 and c.rocfft_cleanup() == 0 and c.rocfft_setup() == 0
    # cache stubs
    buf, ln2 = ctypes.c_void_p(), ctypes.c_size_t(5)
    assert c.rocfft_cache_serialize(ctypes.byref(buf), ctypes.byref(ln2)) == 0 and ln2.value == 0
    assert c.rocfft_cache_deserialize(buf, 0) == 0
    assert c.rocfft_cache_buffer_free(buf) == 0


def test_distributed_descriptions_are_rejected(emu):
    c = emu.c
    f = ctypes.c_void_p()
    assert c.rocfft_field_create(ctypes.byref(f)) == 0
    lo = (ctypes.c_size_t * 2)(0, 0)
    hi = (ctypes.c_size_t * 2)(1, 8)
    st = (ctypes.c_size_t * 2)(8, 1)
    b = ctypes.c_void_p()
    assert c.rocfft_brick_create(ctypes.byref(b), lo, hi, st, 2, 0) == 0
    assert c.rocfft_field_add_brick(f, b) == 0
    d = B.PlanDescription(emu)
    assert c.rocfft_plan_description_add_infield(d.handle, f) == 0
    ln = (ctypes.c_size_t * 1)(8)
    h = ctypes.c_void_p()
    assert c.rocfft_plan_create(ctypes.byref(h), 1, 0, 0, 1, ln, 1, d.handle) == B.STATUS_FAILURE
    assert c.rocfft_brick_destroy(b) == 0 and c.rocfft_field_destroy(f) == 0


def test_work_buffer_contract(emu):
    # reference clients/tests/unit_test.cpp:256-345 (N=8191, Bluestein): missing buffer is
    # allocated by execute, a short one is rejected at execute
    n = 8191  # double precision: three Bluestein kernels and a work buffer
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.DOUBLE, [n], 1, lib=emu)
    need = plan.work_buffer_size
    assert need > 0
    x = np.zeros(n, dtype=np.complex128)
    x[1] = 1
    y = np.zeros_like(x)
    plan.execute([x.ctypes.data], [y.ctypes.data])  # auto-allocated
    assert np.allclose(y, np.exp(-2j * np.pi * np.arange(n) / n), atol=1e-4)
    info = B.ExecutionInfo(emu)
    small = np.zeros(need // 2, dtype=np.uint8)
    info.set_work_buffer(small.ctypes.data, need // 2)
    assert plan.execute_status([x.ctypes.data], [y.ctypes.data], info) == B.STATUS_INVALID_WORK_BUFFER
    big = np.zeros(need, dtype=np.uint8)
    info.set_work_buffer(big.ctypes.data, need)
    y[:] = 0
    assert plan.execute_status([x.ctypes.data], [y.ctypes.data], info) == 0
    assert np.allclose(y, np.exp(-2j * np.pi * np.arange(n) / n), atol=1e-4)


def test_description_is_copied_and_reusable(emu):
    # reference clients/tests/unit_test.cpp:104-193
    n, batch = 64, 2
    x = H.make_input(B.COMPLEX_FORWARD, [n], batch)
    d = B.PlanDescription(emu)
    d.set_data_layout(B.COMPLEX_INTERLEAVED, B.COMPLEX_INTERLEAVED, in_strides=[2], in_distance=2 * n + 3)
    p1 = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.DOUBLE, [n], batch, d, lib=emu)
    # change the description afterwards: the first plan must not notice
    d.set_data_layout(B.COMPLEX_INTERLEAVED, B.COMPLEX_INTERLEAVED, in_strides=[1], in_distance=n)
    p2 = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.DOUBLE, [n], batch, d, lib=emu)
    d.destroy()
    a = np.zeros(batch * (2 * n + 3), dtype=np.complex128)
    for b in range(batch):
        a[b * (2 * n + 3):b * (2 * n + 3) + 2 * n:2] = x[b]
    y1 = np.zeros((batch, n), dtype=np.complex128)
    y2 = np.zeros((batch, n), dtype=np.complex128)
    p1.execute([a.ctypes.data], [y1.ctypes.data])
    xc = np.ascontiguousarray(x)
    p2.execute([xc.ctypes.data], [y2.ctypes.data])
    assert np.array_equal(y1, y2)  # identical bits whatever the input strides
    assert orc.rel_norms(y1, np.fft.fft(x, axis=1))[0] < 1e-15


# ------------------------------------------------------------------ planner
def passes(text):
    return [l for l in text.splitlines() if l.strip().startswith("pass")]


def test_planar_arrays_take_the_compiled_kernels(emu):
    """Every pass that touches a planar array of the user still runs a compiled kernel on its
    branch-free path, whatever the operation fused into it."""
    CP, CI, HP, RE = B.COMPLEX_PLANAR, B.COMPLEX_INTERLEAVED, B.HERMITIAN_PLANAR, B.REAL

    def described(kind, lengths, it, ot, placement=B.NOTINPLACE, prec=B.SINGLE):
        d = B.PlanDescription(emu).set_data_layout(it, ot)
        st, text, _ = emu.describe(placement, kind, prec, lengths, 4, d)
        assert st == 0, (kind, lengths)
        return passes(text)

    for n in (350, 1000, 4096, 10000):
        (p,) = described(B.COMPLEX_FORWARD, [n], CP, CP)
        assert " lean planar_in planar_out" in p and " fast" in p, p
        (p,) = described(B.COMPLEX_INVERSE, [n], CP, CI, prec=B.DOUBLE if n <= 4096 else B.SINGLE)
        assert " lean planar_in " in p and "planar_out" not in p and " fast" in p, p
        (p,) = described(B.COMPLEX_FORWARD, [n], CP, CP, placement=B.INPLACE)
        assert " lean planar_in planar_out" in p, p
    # even-length real: the Hermitian side of the fused pre/post-processing; odd lengths; Bluestein
    (p,) = described(B.REAL_FORWARD, [2000], RE, HP)
    assert " lean planar_out" in p and " fast" in p, p
    (p,) = described(B.REAL_INVERSE, [2000], HP, RE)
    assert " lean planar_in" in p and " fast" in p, p
    (p,) = described(B.REAL_FORWARD, [1001], RE, HP)
    assert " lean planar_out" in p and " fast" in p, p
    (p,) = described(B.REAL_INVERSE, [1001], HP, RE)
    assert " lean planar_in" in p and " fast" in p, p
    (p,) = described(B.COMPLEX_FORWARD, [173], CP, CP)
    assert "bluestein" in p and " lean planar_in planar_out" in p, p
    # 2D: the row pass reads the planar input, the column pass writes the planar output
    ps = described(B.COMPLEX_FORWARD, [360, 90], CP, CP)
    assert all(" lean" in p and " fast" in p and "planar" in p for p in ps), ps


def test_real_rows_of_two_samples(emu):
    """Real transforms whose first dimension has two samples need no transform along it: one
    pre/post-processing pass between the user's arrays."""
    st, text, _ = emu.describe(B.NOTINPLACE, B.REAL_FORWARD, B.SINGLE, [2, 91, 135], 4)
    assert st == 0 and len(passes(text)) == 3 and "n=1 " not in text, text
    K = B
    for lengths, batch in (([2], 5), ([2, 7], 3), ([2, 9, 5], 2)):
        for prec in (K.SINGLE, K.DOUBLE):
            H.check(emu, HOST, K.REAL_FORWARD, lengths, batch, prec)
            H.check(emu, HOST, K.REAL_INVERSE, lengths, batch, prec)
            H.check(emu, HOST, K.REAL_FORWARD, lengths, batch, prec, inplace=True, scale=0.5)
            H.check(emu, HOST, K.REAL_INVERSE, lengths, batch, prec, inplace=True, scale=0.25)
        H.check(emu, HOST, K.REAL_FORWARD, lengths, batch, K.DOUBLE, out_type=K.HERMITIAN_PLANAR)
        H.check(emu, HOST, K.REAL_INVERSE, lengths, batch, K.SINGLE, in_type=K.HERMITIAN_PLANAR, scale=2.0)


def test_short_rows_fold_the_batch_into_the_tile_axis(emu):
    """A column pass over rows shorter than a tile takes (column, batch item) pairs as tile
    entries; results through the run-time-schedule kernel of the emulated runtime."""
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [4, 5], 1000)
    assert st == 0 and "folded(4)" in text and "tile 64x5" in text, text
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [4, 5, 6], 100)
    assert st == 0 and "folded(4)" in text and "folded(20)" in text, text
    # rows of 64 and more elements fill a tile by themselves
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [64, 5], 1000)
    assert st == 0 and "folded" not in text, text
    K = B
    for lengths, batch in (([4, 5], 70), ([3, 3], 130), ([5, 7, 3], 9), ([6, 10], 21)):
        H.check(emu, HOST, K.COMPLEX_FORWARD, lengths, batch, K.DOUBLE)
        H.check(emu, HOST, K.COMPLEX_INVERSE, lengths, batch, K.SINGLE, inplace=True)
        H.check(emu, HOST, K.REAL_FORWARD, lengths, batch, K.DOUBLE)
        H.check(emu, HOST, K.REAL_INVERSE, lengths, batch, K.SINGLE, inplace=True)
        total = int(np.prod(lengths))
        strides = [1]
        for v in lengths[:-1]:
            strides.append(strides[-1] * v)
        H.check(emu, HOST, K.COMPLEX_FORWARD, lengths, batch, K.SINGLE, in_strides=strides, in_dist=total + 3,
                out_strides=strides, out_dist=total + 5)
        H.check(emu, HOST, K.COMPLEX_FORWARD, lengths, batch, K.DOUBLE, in_type=K.COMPLEX_PLANAR,
                out_type=K.COMPLEX_PLANAR)


def test_pass_lists_of_the_benchmark_configurations(emu):
    st, text, work = emu.describe(B.INPLACE, B.COMPLEX_FORWARD, B.SINGLE, [4096], 1024)
    assert st == 0 and len(passes(text)) == 1 and work == 0 and "16x16x16" in text
    st, text, work = emu.describe(B.NOTINPLACE, B.REAL_FORWARD, B.SINGLE, [65536], 4096)
    assert st == 0 and len(passes(text)) <= 3 and work == 4096 * 32768 * 8
    st, text, work = emu.describe(B.NOTINPLACE, B.REAL_INVERSE, B.SINGLE, [65536], 4096)
    assert st == 0 and len(passes(text)) <= 3
    st, text, work = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [4096, 4096], 8)
    # the intermediate of the staged column split is kept with a padded row pitch
    assert st == 0 and len(passes(text)) <= 3 and 8 * 4096 * 4096 * 8 <= work <= 1.02 * 8 * 4096 * 4096 * 8
    st, text, work = emu.describe(B.NOTINPLACE, B.REAL_FORWARD, B.DOUBLE, [512, 512, 512], 1)
    assert st == 0 and len(passes(text)) == 3 and work == 0
    st, text, work = emu.describe(B.NOTINPLACE, B.REAL_INVERSE, B.DOUBLE, [512, 512, 512], 1)
    assert st == 0 and len(passes(text)) == 3 and work == 0
    st, text, work = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.DOUBLE, [1000003], 16)
    assert st == 0 and len(passes(text)) == 3 and "bluestein" in text
    # 16 zero-padded signals of 2^21 points, rows of 4096 kept at a padded pitch
    assert 16 * 2 ** 21 * 16 <= work <= 1.01 * 16 * 2 ** 21 * 16


def test_four_pass_split(emu, monkeypatch):
    """Lengths beyond three levels of kernels (5^12, 3^18 in single precision) take one more
    strided pass; ROCFFT_AMD_SPLIT_LEVELS asks for that plan at lengths the checker finishes."""
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [5 ** 12], 1)
    assert st == 0 and len(passes(text)) == 4 and "split4 C" in text, text
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [3 ** 18], 1)
    assert st == 0 and len(passes(text)) == 4, text
    monkeypatch.setenv("ROCFFT_AMD_SPLIT_LEVELS", "4")
    for n in (65536, 3 ** 9, 30030):
        st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.DOUBLE, [n], 2)
        assert st == 0 and len(passes(text)) == 4, text
        H.check(emu, HOST, B.COMPLEX_FORWARD, [n], 2, B.DOUBLE)
        H.check(emu, HOST, B.COMPLEX_INVERSE, [n], 3, B.SINGLE, inplace=True, scale=0.5)
    # a strided dimension of a 2D transform, and three passes where two would do
    H.check(emu, HOST, B.COMPLEX_FORWARD, [6, 4096], 1, B.DOUBLE)
    monkeypatch.setenv("ROCFFT_AMD_SPLIT_LEVELS", "3")
    H.check(emu, HOST, B.COMPLEX_FORWARD, [32768], 2, B.SINGLE)


def test_three_level_chirp_z(emu, monkeypatch):
    """A convolution length beyond 2^26 (a prime above 2^25) splits into three factors: two strided
    passes each way and one launch of the row kernel per block of rows.  ROCFFT_AMD_BLU3=<m1>,<m0>
    asks for that form at lengths the checker finishes."""
    st, text, work = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [33554467], 1)
    assert st == 0, text
    names = [l for l in passes(text)]
    assert len(names) == 4 + 64 and sum("bluestein P3" in l for l in names) == 64, text  # 2^27 = 64 x 512 x 4096
    assert work == 2 ** 27 * 8
    # the largest convolution length, 2^30
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [400000009], 1)
    assert st == 0 and text.startswith("plan: 516 passes"), text[:300]  # 2^30 = 512 x 512 x 4096
    # 2^31 is beyond the 32-bit sample index of the tables
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [536870923], 1)
    assert st != 0
    monkeypatch.setenv("ROCFFT_AMD_BLU3", "8,16")
    for kind, lengths, batch, prec in ((B.COMPLEX_FORWARD, [1009], 3, B.DOUBLE), (B.COMPLEX_INVERSE, [1009], 2, B.SINGLE),
                                       (B.COMPLEX_FORWARD, [521], 4, B.SINGLE), (B.COMPLEX_FORWARD, [1031], 1, B.DOUBLE),
                                       (B.COMPLEX_FORWARD, [5, 1009], 2, B.DOUBLE), (B.COMPLEX_FORWARD, [1009, 3], 2, B.SINGLE),
                                       (B.REAL_FORWARD, [6, 1009], 1, B.DOUBLE)):
        st, text, _ = emu.describe(B.NOTINPLACE, kind, prec, lengths, batch)
        assert st == 0 and "bluestein P3" in text and "bluestein P5" in text, text
        H.check(emu, HOST, kind, lengths, batch, prec)
        H.check(emu, HOST, kind, lengths, batch, prec, inplace=True, scale=0.5)


def test_one_transform_ignores_the_distances(emu):
    """in place, one transform, different input and output distances (the reference's tests do
    this: clients/tests/accuracy_test_adhoc.cpp:84-157)"""
    for kind, lengths, prec in ((B.COMPLEX_FORWARD, [4], B.SINGLE), (B.COMPLEX_INVERSE, [220], B.DOUBLE),
                                (B.COMPLEX_FORWARD, [19, 33], B.DOUBLE)):
        H.check(emu, HOST, kind, lengths, 1, prec, inplace=True, in_dist=2, out_dist=3)


def test_every_tile_fits_the_hardware(emu):
    for kind, lengths, batch, prec in [(0, [n], 3, p) for n in (2, 3, 30, 100, 4096, 8192, 65536, 2 ** 20,
                                                                 1000, 97, 10007, 1000003) for p in (0, 1)] \
            + [(0, [4096, 4096], 8, 0), (2, [512, 512, 512], 1, 1), (0, [100, 90, 80], 2, 1)]:
        st, text, _ = emu.describe(B.NOTINPLACE, kind, prec, lengths, batch)
        assert st == 0, (lengths, text)
        for line in passes(text):
            m = re.search(r"threads (\d+) grid (\d+) lds (\d+)", line)
            if m:
                threads, grid, lds = map(int, m.groups())
                assert threads % 64 == 0 and 64 <= threads <= 512
                assert lds <= 160 * 1024 and grid >= 1


def test_compiled_schedule_list_is_consistent(emu):
    """Every listed length has one schedule, its radices multiply to the length, the thread
    count respects the register budget of 17 values per thread, and the planner uses it."""
    rows = H.fast_schedules()
    assert len(rows) == len({r[0] for r in rows}) and len(rows) > 200
    for n, radix, tf, td in rows:
        assert int(np.prod(radix)) == n and 1 <= len(radix) <= 4
        assert all(r in (2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17) for r in radix)
        need = max(-(-(n // r) // (17 // r)) for r in radix)
        for t in (tf, td):
            assert t == 0 or need <= t <= 1024
    for n, radix, tf, td in rows[::7]:
        st, text, _ = emu.describe(B.NOTINPLACE, 0, 0, [n], 4)
        assert st == 0
        assert ("radix " + "x".join(map(str, radix)) + " ") in text, (n, text)


# the emulation runs the generic kernel on the schedules of the compiled kernels, composite
# radices 6, 9, 10, 12, 14 and 15 and the prime radix 17 included
@pytest.mark.parametrize("n", [6, 9, 10, 12, 18, 36, 60, 81, 90, 100, 120, 125, 243, 250, 360, 480, 729,
                               1000, 1536, 2187, 3000, 3645, 4000, 4032, 17, 34, 289, 1156, 2040, 4046, 4080,
                               1728, 2925, 3360, 2002])
def test_compiled_schedules_on_the_generic_kernel(emu, n):
    H.check(emu, HOST, B.COMPLEX_FORWARD, [n], 3, B.SINGLE)
    H.check(emu, HOST, B.COMPLEX_INVERSE, [n], 2, B.DOUBLE, inplace=True)
    H.check(emu, HOST, B.REAL_FORWARD, [2 * n], 2, B.DOUBLE)
    H.check(emu, HOST, B.REAL_INVERSE, [2 * n], 2, B.SINGLE)


# ------------------------------------------------------------------ numerics through the emulation
SMALL_1D = [1, 2, 3, 4, 5, 7, 8, 9, 16, 25, 30, 49, 64, 100, 128, 256, 512, 1024, 2048, 4096, 8192,
            11, 13, 17, 19, 97, 121, 169, 1001, 2310]


@pytest.mark.parametrize("n", SMALL_1D)
def test_c2c_1d(emu, n):
    for prec in (B.SINGLE, B.DOUBLE):
        for kind in (B.COMPLEX_FORWARD, B.COMPLEX_INVERSE):
            H.check(emu, HOST, kind, [n], 3, prec)
    H.check(emu, HOST, B.COMPLEX_FORWARD, [n], 2, B.DOUBLE, inplace=True)


@pytest.mark.parametrize("n", [2, 4, 6, 8, 10, 16, 18, 30, 64, 256, 1000, 4096, 8192, 3, 5, 9, 15, 17, 21, 34,
                               38, 97, 194, 625])
def test_real_1d(emu, n):
    for prec in (B.SINGLE, B.DOUBLE):
        for kind in (B.REAL_FORWARD, B.REAL_INVERSE):
            H.check(emu, HOST, kind, [n], 3, prec)
            H.check(emu, HOST, kind, [n], 2, prec, inplace=True)


@pytest.mark.parametrize("lengths", [[16384], [32768], [65536], [6000], [2 ** 17], [30030], [10007], [4099],
                                     [2 * 4099]])
def test_long_1d(emu, lengths):
    H.check(emu, HOST, B.COMPLEX_FORWARD, lengths, 2, B.SINGLE)
    H.check(emu, HOST, B.COMPLEX_INVERSE, lengths, 1, B.DOUBLE, inplace=True)
    if lengths[0] % 2 == 0:
        H.check(emu, HOST, B.REAL_FORWARD, lengths, 2, B.DOUBLE)
        H.check(emu, HOST, B.REAL_INVERSE, lengths, 2, B.SINGLE)
        H.check(emu, HOST, B.REAL_FORWARD, lengths, 1, B.SINGLE, inplace=True)
        H.check(emu, HOST, B.REAL_INVERSE, lengths, 1, B.DOUBLE, inplace=True)


@pytest.mark.parametrize("lengths", [[8193], [10007], [19683], [15625], [9999, 3], [3, 9999]])
def test_long_odd_real(emu, lengths):
    """Odd real lengths beyond one kernel go through a complex scratch copy (split or Bluestein
    in between); the first dimension is the real one."""
    H.check(emu, HOST, B.REAL_FORWARD, lengths, 2, B.DOUBLE)
    H.check(emu, HOST, B.REAL_INVERSE, lengths, 2, B.SINGLE)
    if lengths[0] > 8192:
        H.check(emu, HOST, B.REAL_FORWARD, lengths, 2, B.SINGLE, inplace=True, scale=0.25)
        H.check(emu, HOST, B.REAL_INVERSE, lengths, 2, B.DOUBLE, inplace=True)
        st, text, work = emu.describe(B.NOTINPLACE, B.REAL_FORWARD, B.DOUBLE, lengths, 2)
        assert st == 0 and "real rows to complex scratch" in text and "first bins to Hermitian rows" in text
        assert work >= 2 * int(np.prod(lengths)) * 16


@pytest.mark.parametrize("lengths", [[8, 8], [64, 64], [100, 30], [30, 100], [17, 19], [1024, 1024], [4, 2048],
                                     [2048, 4], [8, 8, 8], [16, 8, 4], [4, 8, 16], [30, 20, 10], [128, 32, 8],
                                     [5, 7, 9], [8192, 4], [4, 8192], [64, 64, 64], [2, 2, 2], [1, 8], [8, 1, 4]])
def test_multi_dim(emu, lengths):
    for kind in range(4):
        H.check(emu, HOST, kind, lengths, 2, B.DOUBLE)
        H.check(emu, HOST, kind, lengths, 1, B.SINGLE, inplace=True)


def test_benchmark_shapes_scaled_down(emu):
    # same decompositions as the full-size configurations, small batch
    H.check(emu, HOST, B.COMPLEX_FORWARD, [4096], 4, B.SINGLE, inplace=True)
    H.check(emu, HOST, B.REAL_FORWARD, [65536], 2, B.SINGLE)
    H.check(emu, HOST, B.REAL_INVERSE, [65536], 2, B.SINGLE)
    H.check(emu, HOST, B.COMPLEX_FORWARD, [4096, 64], 1, B.SINGLE)
    H.check(emu, HOST, B.COMPLEX_FORWARD, [64, 4096], 1, B.SINGLE)
    H.check(emu, HOST, B.REAL_FORWARD, [512, 8, 8], 1, B.DOUBLE)
    H.check(emu, HOST, B.REAL_FORWARD, [8, 512, 4], 1, B.DOUBLE)
    H.check(emu, HOST, B.REAL_INVERSE, [8, 4, 512], 1, B.DOUBLE)


def test_bluestein_two_level_matches_direct_bins(emu):
    # prime just above the single-kernel convolution limit -> three-pass chirp-z
    n = 4099
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.DOUBLE, [n], 1)
    assert "Z1" in text and "Z3" in text
    y, x = H.run_transform(emu, HOST, B.COMPLEX_FORWARD, [n], 1, B.DOUBLE)
    for k in (0, 1, 2049, 4098):
        assert abs(y[0, k] - orc.dft_bin(x[0], k)) / np.abs(y).max() < 1e-14


def test_bluestein_takes_a_shorter_convolution_length(emu):
    """Any length >= 2n-1 serves as the convolution length; when one made of compiled kernels is
    at least 30 % shorter than the next power of two the plan uses it: in one kernel (521 ->
    1053 instead of 2048), in the three-kernel form (8209 -> 8 x 2057 instead of 32768) and in a
    strided dimension (2053 -> 64 x 65 instead of 8192).  A length just below a power of two
    keeps the power of two (1000003 -> 2^21, 1553 -> 4096)."""
    def lengths_in(text):
        return [int(v) for v in re.findall(r" n=(\d+) ", text)]
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [521], 8)
    assert st == 0 and len(passes(text)) == 1 and 1041 <= lengths_in(text)[0] < 1434, text
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [8209], 8)
    n = lengths_in(text)
    assert st == 0 and len(n) == 3 and n[0] == n[2] and 16417 <= n[0] * n[1] < 22937, text
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [9, 2053], 2)
    n = lengths_in(text)
    assert st == 0 and len(n) == 4 and n[1] >= 64 and 4105 <= n[1] * n[2] < 5734, text
    st, text, _ = emu.describe(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [1553], 8)
    assert lengths_in(text) == [4096], text
    for kind, lengths, batch, prec in [(B.COMPLEX_FORWARD, [131], 3, B.SINGLE), (B.COMPLEX_INVERSE, [521], 3, B.DOUBLE),
                                       (B.COMPLEX_FORWARD, [2053], 2, B.SINGLE), (B.COMPLEX_FORWARD, [4099], 2, B.SINGLE),
                                       (B.COMPLEX_INVERSE, [4099], 2, B.DOUBLE), (B.COMPLEX_FORWARD, [8209], 2, B.SINGLE),
                                       (B.COMPLEX_FORWARD, [8209], 1, B.DOUBLE), (B.COMPLEX_FORWARD, [9, 2053], 2, B.SINGLE),
                                       (B.COMPLEX_INVERSE, [9, 2053], 1, B.DOUBLE), (B.REAL_FORWARD, [4099], 2, B.SINGLE),
                                       (B.REAL_INVERSE, [4099], 2, B.DOUBLE), (B.REAL_FORWARD, [1042], 2, B.DOUBLE),
                                       (B.REAL_INVERSE, [16418], 1, B.SINGLE), (B.COMPLEX_FORWARD, [20011], 1, B.SINGLE)]:
        H.check(emu, HOST, kind, lengths, batch, prec)
        H.check(emu, HOST, kind, lengths, batch, prec, inplace=True, scale=0.5)


def test_strides_offsets_planar_scale(emu):
    K = B
    # strided + offset 1D
    H.check(emu, HOST, K.COMPLEX_FORWARD, [64], 3, K.DOUBLE, in_strides=[3], in_dist=200, out_strides=[2],
            out_dist=130, in_offsets=[5, 0], out_offsets=[7, 0])
    # batch interleaved with the transform ("column" access: stride = batch, dist = 1)
    H.check(emu, HOST, K.COMPLEX_FORWARD, [128], 8, K.SINGLE, in_strides=[8], in_dist=1, out_strides=[8],
            out_dist=1)
    # planar in and out, with distinct offsets for the two arrays
    H.check(emu, HOST, K.COMPLEX_INVERSE, [30, 4], 2, K.DOUBLE, in_type=K.COMPLEX_PLANAR,
            out_type=K.COMPLEX_PLANAR, in_offsets=[3, 9], out_offsets=[2, 1])
    H.check(emu, HOST, K.COMPLEX_FORWARD, [256], 2, K.SINGLE, in_type=K.COMPLEX_PLANAR,
            out_type=K.COMPLEX_INTERLEAVED)
    H.check(emu, HOST, K.COMPLEX_FORWARD, [4096 * 4], 1, K.SINGLE, in_type=K.COMPLEX_INTERLEAVED,
            out_type=K.COMPLEX_PLANAR)
    # real with planar Hermitian side and padded rows
    H.check(emu, HOST, K.REAL_FORWARD, [32, 6], 2, K.DOUBLE, out_type=K.HERMITIAN_PLANAR)
    H.check(emu, HOST, K.REAL_INVERSE, [32, 6], 2, K.DOUBLE, in_type=K.HERMITIAN_PLANAR)
    H.check(emu, HOST, K.REAL_FORWARD, [20, 6], 2, K.SINGLE, in_strides=[1, 23], in_dist=150,
            out_strides=[1, 13], out_dist=90)
    H.check(emu, HOST, K.REAL_INVERSE, [21, 6], 2, K.SINGLE, in_strides=[2, 30], in_dist=200,
            out_strides=[1, 25], out_dist=160)
    # transposed output request
    H.check(emu, HOST, K.COMPLEX_FORWARD, [16, 8], 2, K.DOUBLE, out_strides=[8, 1], out_dist=128)
    # scale factor on every route that ends a transform
    for kind, lengths in [(0, [64]), (1, [16384]), (2, [64]), (2, [16384]), (3, [64]), (3, [16384]), (0, [97]),
                          (0, [4099]), (0, [8, 8, 8]), (2, [8, 8]), (3, [7, 8])]:
        H.check(emu, HOST, kind, lengths, 2, K.DOUBLE, scale=1.0 / 64)


def test_no_stray_writes(emu):
    # reference clients/tests/accuracy_test_checkstride.cpp: gaps between strided outputs keep
    # their fill pattern
    for kind, lengths, kw in [(0, [64], dict(out_strides=[3], out_dist=250)),
                              (0, [16384], dict(out_strides=[2], out_dist=40000)),
                              (2, [30, 4], dict(out_strides=[2, 40], out_dist=200)),
                              (3, [32, 4], dict(out_strides=[1, 37], out_dist=170)),
                              (0, [97], dict(out_strides=[2], out_dist=300)),
                              (2, [9], dict(out_strides=[3], out_dist=20))]:
        y, x, touched = H.run_transform(emu, HOST, kind, lengths, 2, B.SINGLE, return_buffers=True, **kw)
        for raw, mask in touched:
            assert np.all(raw[~mask[:raw.size]] == H.GUARD), (kind, lengths)
        ref = H.reference(kind, lengths, 2, x, B.SINGLE)
        assert orc.rel_norms(y, ref)[0] < 1e-5


def test_out_of_place_keeps_its_input_except_c2r(emu):
    for kind, lengths in [(0, [64]), (0, [16384]), (0, [97]), (0, [4099]), (2, [64]), (2, [16384]), (0, [8, 8]),
                          (2, [8, 8, 8])]:
        x = H.make_input(kind, lengths, 2)
        dt = np.float64 if kind == 2 else np.complex128
        a = np.ascontiguousarray(x.astype(dt))
        keep = a.copy()
        n_out = (lengths[0] // 2 + 1) * int(np.prod(lengths[1:])) if kind == 2 else int(np.prod(lengths))
        y = np.zeros((2, n_out), dtype=np.complex128)
        B.Plan(B.NOTINPLACE, kind, B.DOUBLE, lengths, 2, lib=emu).execute([a.ctypes.data], [y.ctypes.data])
        assert np.array_equal(a, keep), (kind, lengths)


def test_c2r_ignores_imaginary_dc_and_nyquist(emu):
    # reference clients/tests/hermitian_test.cpp:35-170: bit-identical output
    for n in (8, 8192, 30, 65536, 9):
        h = H.make_input(B.REAL_INVERSE, [n], 1)
        h2 = h.copy()
        h2[0, 0] += 2.5j
        if n % 2 == 0:
            h2[0, -1] -= 1.5j
        y1, _ = H.run_transform(emu, HOST, B.REAL_INVERSE, [n], 1, B.DOUBLE, x=h)
        y2, _ = H.run_transform(emu, HOST, B.REAL_INVERSE, [n], 1, B.DOUBLE, x=h2)
        assert np.array_equal(y1, y2), n
