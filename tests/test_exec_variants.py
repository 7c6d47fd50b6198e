"""Execution paths around the pass list, on the host emulation of the runtime layer: the
buffers a half-precision plan keeps per stream when several threads execute it at once, and
rocfft_amd_execute_static (no allocation, its limit, callbacks, a misaligned work buffer in the
info).  The GPU counterparts are tests/test_half.py, tests/test_callbacks.py and
tests/test_zz_no_alloc.py."""
import ctypes
import threading

import numpy as np

import helpers as H
import rocfft_amd.binding as B
from oracle import oracle as orc


def _malloc_calls(emu):
    emu.c.fftrt_emu_malloc_calls.restype = ctypes.c_long
    return emu.c.fftrt_emu_malloc_calls()


def test_threads_share_one_half_plan(emu):
    """Executions of one half-precision plan from several threads on one stream, each with its own
    arrays: the plan's scratch copies are shared per stream, so copy-in, passes and copy-out of
    one call must not interleave with another's."""
    n, batch, threads, reps = 4096, 64, 4, 30
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.HALF, [n], batch, lib=emu)
    rng = np.random.default_rng(5)
    xs, refs, outs = [], [], []
    for t in range(threads):
        x = rng.uniform(-0.5, 0.5, (batch, n, 2)).astype(np.float16)
        xs.append(x)
        xq = x[..., 0].astype(np.float64) + 1j * x[..., 1].astype(np.float64)
        refs.append(np.fft.fft(xq, axis=1))
        outs.append(np.zeros((batch, n, 2), dtype=np.float16))
    bad = []

    def work(t):
        for _ in range(reps):
            outs[t][:] = 0
            st = plan.execute_status([xs[t].ctypes.data], [outs[t].ctypes.data])
            got = outs[t][..., 0].astype(np.float64) + 1j * outs[t][..., 1].astype(np.float64)
            err = np.linalg.norm(got - refs[t]) / np.linalg.norm(refs[t])
            if st != 0 or not err < 1.5e-3:
                bad.append((t, st, err))

    pool = [threading.Thread(target=work, args=(t,)) for t in range(threads)]
    for th in pool:
        th.start()
    for th in pool:
        th.join()
    assert not bad, bad[:5]


def test_staged_buffers_are_kept_when_the_work_area_changes_hands(emu):
    """An execution with the caller's work buffer followed by one without it (and back): the
    arrays a half-precision plan keeps are never released while the plan lives, and once both
    kinds of call have been seen nothing more is allocated."""
    n = 20011  # chirp-z in three kernels: needs a work area
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.HALF, [n], 2, lib=emu)
    wb = plan.work_buffer_size
    assert wb > 0
    x = np.random.default_rng(3).uniform(-0.5, 0.5, (2, n, 2)).astype(np.float16)
    y = np.zeros_like(x)
    work = np.zeros(wb + 64, dtype=np.uint8)
    info = B.ExecutionInfo(emu).set_work_buffer(work.ctypes.data, wb)
    results = []
    for use_info in (True, False, True, False):
        y[:] = 0
        before = _malloc_calls(emu)
        assert plan.execute_status([x.ctypes.data], [y.ctypes.data], info if use_info else None) == 0
        results.append((y.copy(), _malloc_calls(emu) - before))
    for got, _ in results[1:]:
        assert np.array_equal(got, results[0][0])
    assert results[2][1] == 0 and results[3][1] == 0, [r[1] for r in results]


def test_execute_static_allocates_nothing(emu):
    # two passes through a work area: the same result as rocfft_execute, no allocation
    n, batch = 1 << 17, 2
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [n], batch, lib=emu)
    assert 0 < plan.work_buffer_size <= B.STATIC_WORK_BYTES
    x = H.make_input(B.COMPLEX_FORWARD, [n], batch).astype(np.complex64)
    want, got = np.zeros_like(x), np.zeros_like(x)
    plan.execute([x.ctypes.data], [want.ctypes.data])
    before = _malloc_calls(emu)
    plan.execute_static([x.ctypes.data], [got.ctypes.data])
    assert _malloc_calls(emu) == before
    assert np.array_equal(want, got)
    ref = orc.transform(orc.COMPLEX_FORWARD, [n], batch, x.astype(np.complex128))
    l2, linf = orc.rel_norms(got.reshape(-1), ref)
    assert l2 <= 1e-5 and linf <= 1e-5

    # a misaligned work buffer in the info is ignored: the pass list is chosen for the static
    # array (8-byte aligned data, 4-byte aligned work buffer in the info)
    work = np.zeros(plan.work_buffer_size + 64, dtype=np.uint8)
    info = B.ExecutionInfo(emu).set_work_buffer(work.ctypes.data + 4, plan.work_buffer_size)
    got2 = np.zeros_like(x)
    before = _malloc_calls(emu)
    plan.execute_static([x.ctypes.data], [got2.ctypes.data], info)
    assert _malloc_calls(emu) == before
    assert np.array_equal(want, got2)
    assert not work.any()  # untouched


def test_execute_static_refusals(emu):
    # beyond the static area: refused, nothing written
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [4096, 4096], 1, lib=emu)
    assert plan.work_buffer_size > B.STATIC_WORK_BYTES
    x = np.zeros((4096, 4096), dtype=np.complex64)
    y = np.full_like(x, 7.0)
    assert plan.execute_static_status([x.ctypes.data], [y.ctypes.data]) == B.STATUS_INVALID_WORK_BUFFER
    assert (y == 7.0).all()
    # half precision whose arrays go through converted copies (the emulation has no converting
    # kernels): the copies would have to be allocated
    half = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.HALF, [256], 4, lib=emu)
    xh = np.zeros((4, 256, 2), dtype=np.float16)
    yh = np.zeros_like(xh)
    before = _malloc_calls(emu)
    assert half.execute_static_status([xh.ctypes.data], [yh.ctypes.data]) == B.STATUS_FAILURE
    assert _malloc_calls(emu) == before
    # ... unless an ordinary execution on the same stream has allocated them already
    assert half.execute_status([xh.ctypes.data], [yh.ctypes.data]) == 0
    before = _malloc_calls(emu)
    assert half.execute_static_status([xh.ctypes.data], [yh.ctypes.data]) == 0
    assert _malloc_calls(emu) == before


def test_execute_static_with_callbacks(emu):
    """callbacks that the first and last kernel call themselves need no staged copy: accepted"""
    from test_callbacks import S_LOAD, S_STORE, callback_library, make_hook

    cblib = callback_library("libcb_host.so")
    n, batch = 1 << 17, 2
    kind, prec = B.COMPLEX_FORWARD, B.SINGLE
    plan = B.Plan(B.NOTINPLACE, kind, prec, [n], batch, lib=emu)
    x = H.make_input(kind, [n], batch).astype(np.complex64)
    got = np.zeros_like(x)
    info = B.ExecutionInfo(emu)
    keep = make_hook(cblib, kind, prec, "load+store")(info, H.HostBackend(), np.float32)
    before = _malloc_calls(emu)
    assert plan.execute_static_status([x.ctypes.data], [got.ctypes.data], info) == 0
    assert _malloc_calls(emu) == before
    ref = orc.transform(orc.COMPLEX_FORWARD, [n], batch, x.astype(np.complex128)) * (S_LOAD * S_STORE)
    l2, linf = orc.rel_norms(got.reshape(-1), ref)
    assert l2 <= 1e-5 and linf <= 1e-5, (l2, linf)
    del keep
