"""Load/store callbacks (reference library/include/rocfft/rocfft.h:533-612): the callbacks of
tests/cb scale every element on the way in and on the way out, so the result must equal
s_load * s_store * transform(x), and an out-of-place transform must leave its input alone."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

import helpers as H
import rocfft_amd.binding as B
from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
S_LOAD, S_STORE = 0.75, -1.5

CASES = [
    (B.COMPLEX_FORWARD, [64], 3, B.SINGLE, {}),
    (B.COMPLEX_INVERSE, [100, 6], 2, B.DOUBLE, {"inplace": True}),
    (B.REAL_FORWARD, [128], 3, B.DOUBLE, {}),
    (B.REAL_FORWARD, [30, 4], 2, B.SINGLE, {"inplace": True}),
    (B.REAL_INVERSE, [64, 8], 2, B.SINGLE, {}),
    (B.REAL_INVERSE, [15], 3, B.DOUBLE, {"inplace": True}),
    (B.COMPLEX_FORWARD, [16384], 2, B.SINGLE, {}),
    (B.COMPLEX_FORWARD, [97], 2, B.DOUBLE, {"in_strides": [2], "in_dist": 200, "out_strides": [3], "out_dist": 300,
                                            "in_offsets": [5, 0], "out_offsets": [2, 0]}),
]


def callback_library(name):
    path = os.path.join(ROOT, "tests", "cb", name)
    if not os.path.exists(path):
        subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "tests", "cb")])
    lib = ctypes.CDLL(path)
    lib.cb_get.restype = ctypes.c_void_p
    lib.cb_get.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int]
    return lib


def make_hook(cblib, kind, precision, which):
    in_complex = kind != B.REAL_FORWARD
    out_complex = kind != B.REAL_INVERSE

    def hook(info, backend, rt):
        keep = []
        for use, is_store, cplx, value in (("load" in which, 0, in_complex, S_LOAD),
                                           ("store" in which, 1, out_complex, S_STORE)):
            if not use:
                continue
            fn = cblib.cb_get(is_store, 1 if cplx else 0, 1 if precision == B.DOUBLE else 0)
            assert fn
            data = backend.alloc(64)
            backend.scatter(data, rt, np.array([0]), np.array([value], dtype=rt))
            keep.append(data)
            (info.set_store_callback if is_store else info.set_load_callback)(fn, backend.ptr(data))
        return keep
    return hook


def check_case(lib, backend, cblib, kind, lengths, batch, precision, kw, which):
    y, x = H.run_transform(lib, backend, kind, lengths, batch, precision,
                           info_hook=make_hook(cblib, kind, precision, which), **kw)
    factor = (S_LOAD if "load" in which else 1.0) * (S_STORE if "store" in which else 1.0)
    ref = H.reference(kind, lengths, batch, x, precision) * factor
    l2, linf = orc.rel_norms(y.reshape(-1), ref.reshape(-1))
    tol = H.tolerance(precision)
    assert l2 <= tol and linf <= tol, (kind, lengths, precision, kw, which, l2, linf)


@pytest.mark.parametrize("which", ["load", "store", "load+store"])
def test_callbacks_through_the_emulation(emu, which):
    cblib = callback_library("libcb_host.so")
    for kind, lengths, batch, precision, kw in CASES:
        check_case(emu, H.HostBackend(), cblib, kind, lengths, batch, precision, kw, which)


def test_callbacks_run_inside_the_kernels(emu):
    """no staged copies: an execution with callbacks makes no device allocation (the plan needs
    no work area here), and the plan's pass count does not depend on callbacks"""
    cblib = callback_library("libcb_host.so")
    emu.c.fftrt_emu_malloc_calls.restype = ctypes.c_long
    for kind, lengths, batch, precision, kw in CASES:
        if kw.get("inplace"):
            continue
        before = []

        def hook(info, backend, rt, _inner=make_hook(cblib, kind, precision, "load+store")):
            keep = _inner(info, backend, rt)
            before.append(emu.c.fftrt_emu_malloc_calls())  # plan and tables exist by now
            return keep

        H.run_transform(emu, H.HostBackend(), kind, lengths, batch, precision, info_hook=hook, **kw)
        after = emu.c.fftrt_emu_malloc_calls()
        st, text, work = emu.describe(B.NOTINPLACE, kind, precision, lengths, batch)
        if work == 0:
            assert after == before[0], (kind, lengths, text)


def test_callback_rules(emu):
    info = B.ExecutionInfo(emu)
    fn = (ctypes.c_void_p * 1)(1)
    c = emu.c
    # shared memory for callbacks is not supported (reference library/src/transform.cpp:80-81)
    assert c.rocfft_execution_info_set_load_callback(info.handle, fn, None, 8) == B.STATUS_INVALID_ARG_VALUE
    # planar arrays cannot be combined with callbacks
    cblib = callback_library("libcb_host.so")
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [16], 1,
                  B.PlanDescription(emu).set_data_layout(B.COMPLEX_PLANAR, B.COMPLEX_PLANAR), lib=emu)
    info.set_load_callback(cblib.cb_get(0, 1, 0), None)
    a = np.zeros(64, dtype=np.float32)
    assert plan.execute_status([a.ctypes.data, a.ctypes.data], [a.ctypes.data, a.ctypes.data], info) == B.STATUS_FAILURE
    # clearing the callback makes the same info usable again
    info.set_load_callback(None)
    re, im, ore, oim = (np.zeros(16, dtype=np.float32) for _ in range(4))
    assert plan.execute_status([re.ctypes.data, im.ctypes.data], [ore.ctypes.data, oim.ctypes.data], info) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["load", "store", "load+store"])
def test_callbacks_on_the_gpu(gpu_lib, which):
    cblib = callback_library("libcb_device.so")
    for kind, lengths, batch, precision, kw in CASES:
        print("callback case", kind, lengths, precision, kw, which, flush=True)
        check_case(gpu_lib, H.TorchBackend(), cblib, kind, lengths, batch, precision, kw, which)


@pytest.mark.gpu
def test_callbacks_and_half_precision_replay_from_a_graph(gpu_lib):
    """Callbacks are called from inside the first and last kernel of the plan: an execution
    with callbacks allocates nothing and can be captured into a graph straight away, and so can
    a half-precision plan whose one kernel converts on load and store.  A half-precision plan of
    several kernels keeps its single-precision intermediate array per stream: the first execution
    on a stream allocates it (so it cannot be the captured one), later ones allocate nothing.
    Every replay is checked against an eager result, with eager work between the replays."""
    import torch

    lib = gpu_lib
    dev = torch.device("cuda:0")
    cblib = callback_library("libcb_device.so")
    gen = torch.Generator(device=dev).manual_seed(3)
    scales = torch.tensor([S_LOAD, S_STORE], dtype=torch.float32, device=dev)
    side = torch.cuda.Stream()
    # one kernel (4096), a split into two (2^17: the callbacks sit in different kernels), and
    # the one-workgroup kernel's length (32768: the run-time-schedule pass list takes over)
    for n, batch in ((4096, 6), (1 << 17, 2), (32768, 3)):
        x = torch.view_as_complex(torch.rand((batch, n, 2), generator=gen, device=dev) - 0.5)
        plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [n], batch, lib=lib)
        info = B.ExecutionInfo(lib).set_stream(side.cuda_stream)
        info.set_load_callback(cblib.cb_get(0, 1, 0), scales[0:].data_ptr())
        info.set_store_callback(cblib.cb_get(1, 1, 0), scales[1:].data_ptr())
        wb = plan.work_buffer_size
        if wb:
            work = torch.empty(wb, dtype=torch.uint8, device=dev)
            info.set_work_buffer(work.data_ptr(), wb)
        xin = x.clone()
        y = torch.zeros_like(x)
        ref = torch.fft.fft(x, dim=1) * (S_LOAD * S_STORE)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                plan.execute([xin.data_ptr()], [y.data_ptr()], info)  # the first execution of this plan
        torch.cuda.synchronize()
        for rep in range(3):
            xin.copy_(x * (rep + 2))
            y.zero_()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            err = (torch.linalg.vector_norm(y - ref * (rep + 2)) / torch.linalg.vector_norm(ref)).item()
            assert err < 1e-5 * (rep + 2), (n, rep, err)
        assert torch.equal(xin, x * 4), n  # out of place: the input is left alone

    # half precision, one kernel that reads and writes the half arrays itself: no scratch copy,
    # the first execution can be the captured one
    hplan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.HALF, [256], 4, lib=lib)
    xh = (torch.rand((4, 256, 2), generator=gen, device=dev) - 0.5).to(torch.float16)
    yh = torch.zeros_like(xh)
    hinfo = B.ExecutionInfo(lib).set_stream(side.cuda_stream)
    torch.cuda.synchronize()
    gh = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(gh, stream=side):
            first = hplan.execute_status([xh.data_ptr()], [yh.data_ptr()], hinfo)
    assert first == 0
    torch.cuda.synchronize()
    xq = torch.view_as_complex(xh.to(torch.float32).contiguous())
    href = torch.view_as_real(torch.fft.fft(xq, dim=1))
    for rep in range(2):
        yh.zero_()
        torch.cuda.synchronize()
        gh.replay()
        torch.cuda.synchronize()
        err = (torch.linalg.vector_norm(yh.to(torch.float32) - href) / torch.linalg.vector_norm(href)).item()
        assert err < 1.5e-3, (rep, err)

    # half precision with a single-precision intermediate array (two kernels): the plan keeps it
    # per stream, the first execution on a stream allocates it (so it cannot be the captured
    # one), later ones allocate nothing
    hplan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.HALF, [256, 256], 2, lib=lib)
    xh = (torch.rand((2, 256 * 256, 2), generator=gen, device=dev) - 0.5).to(torch.float16)
    yh = torch.zeros_like(xh)
    torch.cuda.synchronize()
    g0 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g0, stream=side):
            refused = hplan.execute_status([xh.data_ptr()], [yh.data_ptr()], hinfo)
    assert refused == B.STATUS_FAILURE
    hplan.execute([xh.data_ptr()], [yh.data_ptr()], hinfo)
    side.synchronize()
    want = yh.clone()
    gh = torch.cuda.CUDAGraph()
    yh.zero_()
    with torch.cuda.stream(side):
        with torch.cuda.graph(gh, stream=side):
            hplan.execute([xh.data_ptr()], [yh.data_ptr()], hinfo)
    torch.cuda.synchronize()
    for rep in range(2):
        yh.zero_()
        torch.cuda.synchronize()
        gh.replay()
        torch.cuda.synchronize()
        assert torch.equal(yh, want), rep
