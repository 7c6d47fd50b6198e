"""Shared machinery of the parity tests: lays a logical input out in memory as a
plan description asks, runs the plan through the C ABI, gathers the output back
and compares with the CPU checker.  `backend` hides where the buffers live:
host memory for the emulated runtime, torch CUDA tensors for the real one."""
import numpy as np

import rocfft_amd.binding as B
from oracle import oracle as orc

GUARD = 0xCD


def element_indices(lengths, batch, strides, dist, offset):
    """flat element index of every (batch, ..., i1, i0), shape (batch, prod(lengths)); i0 fastest."""
    idx = np.zeros(1, dtype=np.int64)
    for n, s in zip(lengths, strides):
        # each new dimension is slower than the ones already laid out
        idx = (idx[None, :] + (np.arange(n, dtype=np.int64) * s)[:, None]).reshape(-1)
    b = np.arange(batch, dtype=np.int64) * dist
    return offset + b[:, None] + idx[None, :]


class HostBackend:
    """buffers are numpy arrays (emulated runtime)"""

    def alloc(self, nbytes):
        return np.full(nbytes, GUARD, dtype=np.uint8)

    def ptr(self, buf):
        return buf.ctypes.data

    def write(self, buf, byte_offset, arr):
        raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
        buf[byte_offset:byte_offset + raw.size] = raw

    def scatter(self, buf, dtype, index, values):
        buf.view(dtype)[index.reshape(-1)] = values.reshape(-1).astype(dtype)

    def gather(self, buf, dtype, index):
        return buf.view(dtype)[index.reshape(-1)].reshape(index.shape)

    def to_numpy(self, buf):
        return buf

    def sync(self):
        pass


class TorchBackend:
    """buffers are uint8 CUDA tensors"""

    def __init__(self):
        import torch

        self.torch = torch
        self.dev = torch.device("cuda:0")

    def alloc(self, nbytes):
        return self.torch.full((nbytes,), GUARD, dtype=self.torch.uint8, device=self.dev)

    def ptr(self, buf):
        return buf.data_ptr()

    def scatter(self, buf, dtype, index, values):
        host = np.full(buf.numel(), GUARD, dtype=np.uint8)
        host.view(dtype)[index.reshape(-1)] = values.reshape(-1).astype(dtype)
        buf.copy_(self.torch.from_numpy(host))

    def gather(self, buf, dtype, index):
        return buf.cpu().numpy().view(dtype)[index.reshape(-1)].reshape(index.shape)

    def to_numpy(self, buf):
        return buf.cpu().numpy()

    def sync(self):
        self.torch.cuda.synchronize()


def _is_planar(t):
    return t in (B.COMPLEX_PLANAR, B.HERMITIAN_PLANAR)


def default_types(kind):
    if kind in (B.COMPLEX_FORWARD, B.COMPLEX_INVERSE):
        return B.COMPLEX_INTERLEAVED, B.COMPLEX_INTERLEAVED
    if kind == B.REAL_FORWARD:
        return B.REAL, B.HERMITIAN_INTERLEAVED
    return B.HERMITIAN_INTERLEAVED, B.REAL


def default_layout(kind, lengths, inplace):
    """(in_lengths, out_lengths, in_strides, in_dist, out_strides, out_dist) per rocfft defaults."""
    ilen, olen = list(lengths), list(lengths)
    if kind == B.REAL_FORWARD:
        olen[0] = lengths[0] // 2 + 1
    if kind == B.REAL_INVERSE:
        ilen[0] = lengths[0] // 2 + 1

    def contiguous(ln):
        s = [1]
        for v in ln[:-1]:
            s.append(s[-1] * v)
        return s, s[-1] * ln[-1]

    istr, idist = contiguous(ilen)
    ostr, odist = contiguous(olen)
    if inplace and kind == B.REAL_FORWARD:
        row = 2 * olen[0]
        istr, idist = contiguous([row] + ilen[1:])
    if inplace and kind == B.REAL_INVERSE:
        row = 2 * ilen[0]
        ostr, odist = contiguous([row] + olen[1:])
    return ilen, olen, istr, idist, ostr, odist


def make_input(kind, lengths, batch, seed=1):
    import inputs

    total = int(np.prod(lengths))
    if kind in (B.COMPLEX_FORWARD, B.COMPLEX_INVERSE):
        return inputs.complex_input(seed, 0, total * batch).reshape(batch, total)
    x = inputs.real_input(seed, 0, total * batch).reshape(batch, total)
    if kind == B.REAL_FORWARD:
        return x
    # a valid Hermitian input: the forward transform of real data
    return orc.transform(orc.REAL_FORWARD, lengths, batch, x, ld=True).reshape(batch, -1)


def run_transform(lib, backend, kind, lengths, batch, precision, inplace=False, in_type=None,
                  out_type=None, in_strides=None, in_dist=0, out_strides=None, out_dist=0,
                  in_offsets=None, out_offsets=None, scale=None, x=None, seed=1, use_work_buffer=True,
                  stream=None, return_buffers=False, info_hook=None):
    """Runs one plan; returns (output as (batch, n_out) float64/complex128, reference input used)."""
    rt = np.float32 if precision == B.SINGLE else np.float64
    dit, dot = default_types(kind)
    in_type = dit if in_type is None else in_type
    out_type = dot if out_type is None else out_type
    ilen, olen, distr, didist, dostr, dodist = default_layout(kind, lengths, inplace)
    istr = list(in_strides) if in_strides else distr
    ostr = list(out_strides) if out_strides else dostr
    idist = in_dist or (didist if not in_strides else ilen[-1] * istr[-1])
    odist = out_dist or (dodist if not out_strides else olen[-1] * ostr[-1])
    ioff = list(in_offsets) if in_offsets else [0, 0]
    ooff = list(out_offsets) if out_offsets else [0, 0]
    if x is None:
        x = make_input(kind, lengths, batch, seed)

    custom = (in_strides or out_strides or in_dist or out_dist or in_offsets or out_offsets
              or in_type != dit or out_type != dot or scale is not None)
    desc = None
    if custom:
        desc = B.PlanDescription(lib)
        desc.set_data_layout(in_type, out_type, ioff if in_offsets else None, ooff if out_offsets else None,
                             istr if in_strides else None, in_dist, ostr if out_strides else None, out_dist)
        if scale is not None:
            desc.set_scale_factor(scale)
    plan = B.Plan(B.INPLACE if inplace else B.NOTINPLACE, kind, precision, lengths, batch, desc, lib=lib)

    in_real = in_type == B.REAL
    out_real = out_type == B.REAL
    sc = np.dtype(rt).itemsize
    in_idx = element_indices(ilen, batch, istr, idist, 0)
    out_idx = element_indices(olen, batch, ostr, odist, 0)
    in_elems = int(in_idx.max()) + 1 + max(ioff)
    out_elems = int(out_idx.max()) + 1 + max(ooff)
    in_esize = sc if (in_real or _is_planar(in_type)) else 2 * sc
    out_esize = sc if (out_real or _is_planar(out_type)) else 2 * sc
    pad = 64
    if inplace:
        nbytes = max(in_elems * in_esize, out_elems * out_esize) + pad
        in_bufs = [backend.alloc(nbytes)]
        if _is_planar(in_type):
            in_bufs.append(backend.alloc(nbytes))
        out_bufs = in_bufs
    else:
        in_bufs = [backend.alloc(in_elems * in_esize + pad) for _ in range(2 if _is_planar(in_type) else 1)]
        out_bufs = [backend.alloc(out_elems * out_esize + pad) for _ in range(2 if _is_planar(out_type) else 1)]

    ct = np.complex64 if precision == B.SINGLE else np.complex128
    if in_real:
        backend.scatter(in_bufs[0], rt, in_idx + ioff[0], x)
    elif _is_planar(in_type):
        backend.scatter(in_bufs[0], rt, in_idx + ioff[0], x.real)
        backend.scatter(in_bufs[1], rt, in_idx + ioff[1], x.imag)
    else:
        backend.scatter(in_bufs[0], ct, in_idx + ioff[0], x)

    info = B.ExecutionInfo(lib)
    work = None
    wb = plan.work_buffer_size
    if wb and use_work_buffer:
        work = backend.alloc(wb)
        info.set_work_buffer(backend.ptr(work), wb)
    if stream is not None:
        info.set_stream(stream)
    hook_state = info_hook(info, backend, rt) if info_hook else None  # kept alive until the result is read
    plan.execute([backend.ptr(b) for b in in_bufs],
                 None if inplace else [backend.ptr(b) for b in out_bufs], info)
    backend.sync()

    if out_real:
        y = backend.gather(out_bufs[0], rt, out_idx + ooff[0]).astype(np.float64)
    elif _is_planar(out_type):
        y = backend.gather(out_bufs[0], rt, out_idx + ooff[0]).astype(np.float64) \
            + 1j * backend.gather(out_bufs[1], rt, out_idx + ooff[1]).astype(np.float64)
    else:
        y = backend.gather(out_bufs[0], ct, out_idx + ooff[0]).astype(np.complex128)
    if return_buffers:
        touched = []
        for b, off in zip(out_bufs, ooff):
            esz = out_esize
            mask = np.zeros(backend.to_numpy(b).size, dtype=bool)
            starts = ((out_idx.reshape(-1) + off) * esz)
            for k in range(esz):
                mask[starts + k] = True
            touched.append((backend.to_numpy(b), mask))
        return y, x, touched
    del hook_state
    plan.destroy()
    return y, x


def reference(kind, lengths, batch, x, precision, scale=None):
    # the input the library saw was rounded to the plan precision
    if precision == B.SINGLE:
        x = x.astype(np.complex64).astype(np.complex128) if np.iscomplexobj(x) else \
            x.astype(np.float32).astype(np.float64)
    y = orc.transform(kind, lengths, batch, x, ld=(precision == B.DOUBLE))
    if scale is not None:
        y = y * scale
    return y.reshape(batch, -1)


def tolerance(precision):
    """north-star bar: relative L2 and Linf <= 1e-5 (single) / 1e-13 (double)."""
    return 1e-5 if precision == B.SINGLE else 1e-13


def check(lib, backend, kind, lengths, batch, precision, **kw):
    y, x = run_transform(lib, backend, kind, lengths, batch, precision, **kw)
    ref = reference(kind, lengths, batch, x, precision, kw.get("scale"))
    l2, linf = orc.rel_norms(y.reshape(-1), ref.reshape(-1))
    tol = tolerance(precision)
    assert l2 <= tol and linf <= tol, (kind, lengths, batch, precision, kw, l2, linf)
    return l2, linf


def fast_schedules():
    """[(n, radices, threads single, threads double)] from the list of compile-time-schedule
    kernels (rocfft_amd/csrc/fast_schedules.h); threads 0 = the fewest possible"""
    import os
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "rocfft_amd", "csrc", "fast_schedules.h")).read()
    out = []
    for m in re.finditer(r"^FAST_SCHED\(([\d, ]+)\)", text, re.M):
        v = [int(a) for a in m.group(1).split(",")]
        out.append((v[2], [r for r in v[3:7] if r > 1], v[7], v[8]))
    return out
