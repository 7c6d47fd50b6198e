"""rocfft_amd_execute_static, the execute variant that allocates nothing: its work
area is a device array the library holds for the life of the process.  Called
through the C ABI and compared with rocfft_execute (which allocates a work
buffer per call) on the same inputs: the two run the same kernels, so the
outputs have to be bit-identical.  Two calls in a row share the one array, the
second with a smaller input; then a plan beyond the limit is refused.
"""
import numpy as np
import pytest

import inputs
import rocfft_amd.binding as B

pytestmark = pytest.mark.gpu


def _complex_input(torch, dev, seed, batch, n, dtype):
    real = torch.float32 if dtype == torch.complex64 else torch.float64
    x = inputs.torch_uniform01(torch, dev, seed, 0, 2 * n * batch).to(real) - 0.5
    return torch.view_as_complex(x.reshape(batch, n, 2).contiguous())


def _both_ways(torch, plan, x):
    """(output of rocfft_execute, output of rocfft_amd_execute_static), each on a poisoned buffer"""
    want = torch.full_like(x, float("nan"))
    got = torch.full_like(x, float("nan"))
    plan.execute([x.data_ptr()], [want.data_ptr()])
    torch.cuda.synchronize()
    plan.execute_static([x.data_ptr()], [got.data_ptr()])
    torch.cuda.synchronize()
    return want, got


def test_static_work_area_matches_execute(gpu_lib):
    import torch

    lib = gpu_lib
    dev = torch.device("cuda:0")
    # first call: 2^17 points x 16, two passes through 16 MiB of the work area
    big = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [1 << 17], 16, lib=lib)
    assert 0 < big.work_buffer_size <= B.STATIC_WORK_BYTES
    x1 = _complex_input(torch, dev, 11, 16, 1 << 17, torch.complex64)
    want1, got1 = _both_ways(torch, big, x1)
    assert torch.isfinite(torch.view_as_real(got1)).all()
    assert torch.equal(torch.view_as_real(want1), torch.view_as_real(got1))
    # and it is the transform: against the library's own one-kernel path is no check, so
    # compare a few rows with numpy in double precision
    ref = np.fft.fft(x1[:2].cpu().numpy().astype(np.complex128), axis=1)
    err = np.linalg.norm(got1[:2].cpu().numpy() - ref) / np.linalg.norm(ref)
    assert err < 1e-5, err

    # second call right behind it, smaller, a different kind of plan (chirp-z in double
    # precision: three kernels that use the start of the same array)
    n2 = 20011
    small = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.DOUBLE, [n2], 8, lib=lib)
    assert 0 < small.work_buffer_size < big.work_buffer_size
    x2 = _complex_input(torch, dev, 12, 8, n2, torch.complex128)
    want2, got2 = _both_ways(torch, small, x2)
    assert torch.isfinite(torch.view_as_real(got2)).all()
    assert torch.equal(torch.view_as_real(want2), torch.view_as_real(got2))
    ref = np.fft.fft(x2[:2].cpu().numpy(), axis=1)
    err = np.linalg.norm(got2[:2].cpu().numpy() - ref) / np.linalg.norm(ref)
    assert err < 1e-13, err

    # the first plan again: what the second call left in the array does not matter
    want3, got3 = _both_ways(torch, big, x1)
    assert torch.equal(torch.view_as_real(want1), torch.view_as_real(got3))

    # a plan without a work area runs as well; a stream set in the info is used
    one = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [4096], 8, lib=lib)
    assert one.work_buffer_size == 0
    x4 = _complex_input(torch, dev, 13, 8, 4096, torch.complex64)
    s = torch.cuda.Stream()
    info = B.ExecutionInfo(lib).set_stream(s.cuda_stream)
    y4 = torch.empty_like(x4)
    torch.cuda.synchronize()
    one.execute_static([x4.data_ptr()], [y4.data_ptr()], info)
    s.synchronize()
    ref = torch.fft.fft(x4, dim=1)
    assert (torch.linalg.vector_norm(y4 - ref) / torch.linalg.vector_norm(ref)).item() < 1e-5


def test_static_work_area_limit(gpu_lib):
    import torch

    lib = gpu_lib
    dev = torch.device("cuda:0")
    # 4096 x 4096 needs 135 MB of work area: refused, nothing written
    plan = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [4096, 4096], 1, lib=lib)
    assert plan.work_buffer_size > B.STATIC_WORK_BYTES
    x = torch.zeros((4096, 4096), dtype=torch.complex64, device=dev)
    y = torch.full_like(x, 7.0)
    st = plan.execute_static_status([x.data_ptr()], [y.data_ptr()])
    torch.cuda.synchronize()
    assert st == B.STATUS_INVALID_WORK_BUFFER
    assert (y == 7.0).all()
    # half precision with a single-precision intermediate array, which the plan would have to
    # allocate: refused as well
    half = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.HALF, [256, 256], 2, lib=lib)
    xh = torch.zeros((2, 256 * 256, 2), dtype=torch.float16, device=dev)
    yh = torch.zeros_like(xh)
    assert half.execute_static_status([xh.data_ptr()], [yh.data_ptr()]) == B.STATUS_FAILURE


def test_static_variant_allocates_no_device_memory(gpu_lib):
    """free device memory (as the driver reports it) is the same before and after the calls;
    half-precision and callback plans whose kernels do the conversion / call the callbacks
    themselves are accepted"""
    import torch

    from test_callbacks import S_LOAD, S_STORE, callback_library

    lib = gpu_lib
    dev = torch.device("cuda:0")
    big = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.SINGLE, [1 << 17], 16, lib=lib)
    x = _complex_input(torch, dev, 21, 16, 1 << 17, torch.complex64)
    y = torch.empty_like(x)
    half = B.Plan(B.NOTINPLACE, B.COMPLEX_FORWARD, B.HALF, [1024], 64, lib=lib)
    xh = (torch.view_as_real(_complex_input(torch, dev, 22, 64, 1024, torch.complex64))).to(torch.float16)
    yh = torch.zeros_like(xh)
    cblib = callback_library("libcb_device.so")
    scales = torch.tensor([S_LOAD, S_STORE], dtype=torch.float32, device=dev)
    cinfo = B.ExecutionInfo(lib)
    cinfo.set_load_callback(cblib.cb_get(0, 1, 0), scales[0:].data_ptr())
    cinfo.set_store_callback(cblib.cb_get(1, 1, 0), scales[1:].data_ptr())
    yc = torch.empty_like(x)
    # one warm-up of each kernel (code objects are loaded on first use), then measure
    big.execute_static([x.data_ptr()], [y.data_ptr()])
    half.execute_static([xh.data_ptr()], [yh.data_ptr()])
    big.execute_static([x.data_ptr()], [yc.data_ptr()], cinfo)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        big.execute_static([x.data_ptr()], [y.data_ptr()])
        half.execute_static([xh.data_ptr()], [yh.data_ptr()])
        big.execute_static([x.data_ptr()], [yc.data_ptr()], cinfo)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    ref = torch.fft.fft(x, dim=1)
    assert (torch.linalg.vector_norm(y - ref) / torch.linalg.vector_norm(ref)).item() < 1e-5
    assert (torch.linalg.vector_norm(yc - ref * (S_LOAD * S_STORE)) / torch.linalg.vector_norm(ref)).item() < 2e-5
    href = torch.view_as_real(torch.fft.fft(torch.view_as_complex(xh.to(torch.float32).contiguous()), dim=1))
    err = (torch.linalg.vector_norm(yh.to(torch.float32) - href) / torch.linalg.vector_norm(href)).item()
    assert err < 1.5e-3, err
