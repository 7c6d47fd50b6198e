"""Half-precision plans (rocfft_precision_half): arrays of IEEE half values, arithmetic in single
precision.  On the GPU the first and last pass of a plan read and write the half arrays
themselves where a compiled kernel with that form exists (interleaved or real arrays, lengths
up to 4096 per pass); other sides go through converted copies, as everything does in the
emulation.  The checker transforms the half-rounded input in long double; the
result may differ by the rounding of the output to half (2^-11 relative per element)."""
import numpy as np
import pytest

import rocfft_amd.binding as B
from oracle import oracle as orc

TOL = 1.5e-3  # relative L2 and Linf; half has 11 significant bits


def run_half(lib, alloc, kind, lengths, batch, inplace=False, planar=False):
    """alloc(nbytes) -> (pointer, write(np.ndarray of float16), read() -> np.ndarray of float16)"""
    rng = np.random.default_rng(abs(hash((kind, tuple(lengths), batch, inplace, planar))) % 2 ** 31)
    total = int(np.prod(lengths))
    h0 = lengths[0] // 2 + 1
    htotal = total // lengths[0] * h0
    if kind in (B.COMPLEX_FORWARD, B.COMPLEX_INVERSE):
        x = (rng.uniform(-0.5, 0.5, (batch, total)) + 1j * rng.uniform(-0.5, 0.5, (batch, total)))
        xin = np.stack([x.real, x.imag], -1).astype(np.float16)
        xq = xin[..., 0].astype(np.float64) + 1j * xin[..., 1].astype(np.float64)
        nout, out_complex = total, True
    elif kind == B.REAL_FORWARD:
        xin = rng.uniform(-1, 1, (batch, total)).astype(np.float16)
        xq = xin.astype(np.float64)
        nout, out_complex = htotal, True
    else:
        xr = rng.uniform(-1, 1, (batch, total))
        spec = orc.transform(B.REAL_FORWARD, lengths, batch, xr, ld=True).reshape(batch, htotal) / total
        xin = np.stack([spec.real, spec.imag], -1).astype(np.float16)
        xq = xin[..., 0].astype(np.float64) + 1j * xin[..., 1].astype(np.float64)
        nout, out_complex = total, False
    ref = orc.transform(kind, lengths, batch, xq, ld=True).reshape(batch, nout)

    desc = None
    if planar:
        desc = B.PlanDescription(lib).set_data_layout(B.COMPLEX_PLANAR, B.COMPLEX_PLANAR)
    plan = B.Plan(B.INPLACE if inplace else B.NOTINPLACE, kind, B.HALF, lengths, batch, desc, lib=lib)
    info = B.ExecutionInfo(lib)
    if planar:
        bufs_in = [alloc(xin[..., 0].nbytes), alloc(xin[..., 1].nbytes)]
        bufs_in[0][1](np.ascontiguousarray(xin[..., 0]))
        bufs_in[1][1](np.ascontiguousarray(xin[..., 1]))
        bufs_out = bufs_in if inplace else [alloc(batch * nout * 2), alloc(batch * nout * 2)]
        plan.execute([b[0] for b in bufs_in], None if inplace else [b[0] for b in bufs_out], info)
        got = bufs_out[0][2]()[:batch * nout].astype(np.float64) + 1j * bufs_out[1][2]()[:batch * nout].astype(np.float64)
        got = got.reshape(batch, nout)
    elif inplace and kind in (B.REAL_FORWARD, B.REAL_INVERSE):
        # padded rows of 2 (N/2 + 1) half values
        rows = total // lengths[0] * batch
        buf = np.zeros((rows, 2 * h0), dtype=np.float16)
        if kind == B.REAL_FORWARD:
            buf[:, :lengths[0]] = xin.reshape(rows, lengths[0])
        else:
            buf[:] = xin.reshape(rows, 2 * h0)
        dev = alloc(buf.nbytes)
        dev[1](buf)
        plan.execute([dev[0]], None, info)
        res = dev[2]()[:rows * 2 * h0].reshape(rows, 2 * h0).astype(np.float64)
        got = (res[:, 0::2] + 1j * res[:, 1::2]).reshape(batch, nout) if kind == B.REAL_FORWARD \
            else res[:, :lengths[0]].reshape(batch, nout)
    else:
        dev_in = alloc(xin.nbytes)
        dev_in[1](xin)
        out_bytes = batch * nout * (4 if out_complex else 2)
        dev_out = dev_in if inplace else alloc(out_bytes)
        plan.execute([dev_in[0]], None if inplace else [dev_out[0]], info)
        res = dev_out[2]()[:batch * nout * (2 if out_complex else 1)].astype(np.float64)
        got = (res[0::2] + 1j * res[1::2]).reshape(batch, nout) if out_complex else res.reshape(batch, nout)
    l2, linf = orc.rel_norms(np.asarray(got).reshape(-1), ref.reshape(-1))
    assert l2 <= TOL and linf <= TOL, (kind, lengths, batch, inplace, planar, l2, linf)


def host_alloc(nbytes):
    a = np.zeros(nbytes // 2 + 8, dtype=np.float16)

    def write(v):
        a[:v.size] = v.reshape(-1)
    return a.ctypes.data, write, lambda: a.copy()


def torch_alloc(nbytes):
    import torch
    t = torch.zeros(nbytes // 2 + 8, dtype=torch.float16, device="cuda")

    def write(v):
        t[:v.size] = torch.from_numpy(np.ascontiguousarray(v.reshape(-1))).to("cuda")

    def read():
        torch.cuda.synchronize()
        return t.cpu().numpy()
    return t.data_ptr(), write, read


CASES = [(B.COMPLEX_FORWARD, [64], 3, {}), (B.COMPLEX_INVERSE, [100], 2, {"inplace": True}),
         (B.COMPLEX_FORWARD, [32, 16], 2, {"planar": True}), (B.COMPLEX_FORWARD, [8, 8, 8], 1, {"inplace": True}),
         (B.REAL_FORWARD, [256], 3, {}), (B.REAL_FORWARD, [30, 6], 2, {"inplace": True}),
         (B.REAL_INVERSE, [64, 4], 2, {}), (B.REAL_INVERSE, [15], 3, {"inplace": True}),
         (B.COMPLEX_FORWARD, [4096], 2, {})]


@pytest.mark.parametrize("case", CASES)
def test_half_through_the_emulation(emu, case):
    kind, lengths, batch, kw = case
    run_half(emu, host_alloc, kind, lengths, batch, **kw)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_half_on_the_gpu(gpu_lib, case):
    kind, lengths, batch, kw = case
    run_half(gpu_lib, torch_alloc, kind, lengths, batch, **kw)


# the first and last kernel convert on load / store: one kernel, several passes (the intermediate
# results stay in single precision), in place, short transforms (tile copy), real transforms with
# the fused pre/post-processing, 2D/3D; and sides that fall back to converted copies (planar,
# odd lengths, chirp-z lengths, a first pass longer than 4096 points)
FUSED_CASES = [(B.COMPLEX_FORWARD, [4096], 64, {}), (B.COMPLEX_INVERSE, [4096], 33, {"inplace": True}),
               (B.COMPLEX_FORWARD, [1000], 100, {}), (B.COMPLEX_FORWARD, [8], 5000, {}),
               (B.COMPLEX_INVERSE, [16], 3001, {"inplace": True}), (B.COMPLEX_FORWARD, [65536], 5, {}),
               (B.COMPLEX_INVERSE, [30000], 7, {"inplace": True}), (B.COMPLEX_FORWARD, [1 << 20], 1, {}),
               (B.REAL_FORWARD, [8192], 40, {}), (B.REAL_INVERSE, [8192], 40, {}),
               (B.REAL_FORWARD, [2000], 50, {"inplace": True}), (B.REAL_INVERSE, [2000], 50, {"inplace": True}),
               (B.REAL_FORWARD, [32], 4000, {}), (B.REAL_INVERSE, [32], 4000, {}),
               (B.COMPLEX_FORWARD, [256, 256], 4, {}), (B.COMPLEX_INVERSE, [100, 60], 9, {"inplace": True}),
               (B.REAL_FORWARD, [512, 512], 3, {}), (B.REAL_INVERSE, [512, 512], 3, {}),
               (B.COMPLEX_FORWARD, [64, 64, 64], 2, {}), (B.REAL_FORWARD, [48, 40, 36], 2, {}),
               (B.REAL_INVERSE, [48, 40, 36], 2, {"inplace": True}), (B.COMPLEX_FORWARD, [4, 5], 3000, {}),
               (B.COMPLEX_FORWARD, [360, 360], 2, {"planar": True}), (B.REAL_FORWARD, [1001], 20, {}),
               (B.REAL_INVERSE, [625], 20, {}), (B.COMPLEX_FORWARD, [173], 100, {}),
               (B.COMPLEX_FORWARD, [8192], 10, {}), (B.REAL_FORWARD, [65536], 6, {}),
               (B.REAL_INVERSE, [65536], 6, {})]


@pytest.mark.gpu
@pytest.mark.parametrize("case", FUSED_CASES)
def test_half_arrays_read_and_written_by_the_kernels(gpu_lib, case):
    kind, lengths, batch, kw = case
    run_half(gpu_lib, torch_alloc, kind, lengths, batch, **kw)
