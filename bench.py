#!/usr/bin/env python3
"""Benchmark of the FFT hot path on one MI355X.

One "step" is one pass of the hot path over one batch of synthetic input that
is already resident in HBM: for the default workload (the second benchmark
configuration) a step is the real forward transform of 4096 signals of 65536
float32 samples followed by the real inverse transform of the result, both out
of place, through rocfft_execute of this library's C ABI.

Prints ONE JSON line.  `value` is GFLOP/s in the 5*N*log2(N) convention summed
over the transforms of a step.  `roofline` prices the slowest kernel of the step
against the HBM peak using per-kernel durations taken with HIP events inside this
script; `cpu_baseline` is the fastest CPU figure the host offers for a bounded sample
of the same workload, looked for in the order FFTW (the reference's CPU path), MKL's
FFTW interface, scipy's pocketfft, this repository's own port (`kind` and `chain` say
which was found and used); `cpu_other` holds the remaining ones.
`all_configs` adds one short measurement for each of the five benchmark
configurations next to reference rocFFT, timed through the identical harness (the
same rocfft.h calls on the same buffers, preallocated outputs, caller-owned work
buffer, same warm-up and step count) in a child process per copy of librocfft
found on the box; the torch.fft figure (the same library behind hipFFT, with
PyTorch's allocations inside the timed region) stays as a second column.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak


def workloads():
    """name, transform list [(kind, lengths, batch, precision, inplace)], flops and bytes per step"""
    import rocfft_amd as rf

    def flops(lengths, batch):
        n = 1
        for v in lengths:
            n *= v
        return 5.0 * n * math.log2(n) * batch

    w = {}
    n, b = 4096, 1024
    w[1] = dict(name="c2c_1d_4096_x1024_f32_inplace", dtype="f32",
                transforms=[(rf.COMPLEX_FORWARD, [n], b, rf.SINGLE, True)], flops=flops([n], b),
                bytes=2.0 * n * b * 8)
    n, b = 65536, 4096
    per_dir = n * b * 4 + (n // 2 + 1) * b * 8
    w[2] = dict(name="r2c_c2r_1d_65536_x4096_f32_roundtrip", dtype="f32",
                transforms=[(rf.REAL_FORWARD, [n], b, rf.SINGLE, False), (rf.REAL_INVERSE, [n], b, rf.SINGLE, False)],
                flops=2 * flops([n], b), bytes=2.0 * per_dir)
    n, b = 4096, 8
    w[3] = dict(name="c2c_2d_4096x4096_x8_f32", dtype="f32",
                transforms=[(rf.COMPLEX_FORWARD, [n, n], b, rf.SINGLE, False)], flops=flops([n, n], b),
                bytes=2.0 * n * n * b * 8)
    n = 512
    per_dir = n ** 3 * 8 + n * n * (n // 2 + 1) * 16
    w[4] = dict(name="r2c_c2r_3d_512cubed_f64_roundtrip", dtype="f64",
                transforms=[(rf.REAL_FORWARD, [n, n, n], 1, rf.DOUBLE, False),
                            (rf.REAL_INVERSE, [n, n, n], 1, rf.DOUBLE, False)],
                flops=2 * flops([n, n, n], 1), bytes=2.0 * per_dir)
    n, b = 1000003, 16
    w[5] = dict(name="c2c_1d_prime1000003_x16_f64_bluestein", dtype="f64",
                transforms=[(rf.COMPLEX_FORWARD, [n], b, rf.DOUBLE, False)], flops=flops([n], b),
                bytes=2.0 * n * b * 16)
    return w


class Step:
    """plans, device buffers and execution infos of one workload; run() enqueues one step"""

    def __init__(self, cfg_id, wl, torch, stream_ptr, lib=None):
        import inputs
        import rocfft_amd as rf

        self.torch = torch
        self.rf = rf
        dev = torch.device("cuda:0")
        self.x = inputs.torch_config_input(torch, dev, cfg_id).contiguous()
        self.calls = []
        self.keep = []
        cur = self.x
        for (kind, lengths, batch, prec, inplace) in wl["transforms"]:
            plan = rf.Plan(rf.INPLACE if inplace else rf.NOTINPLACE, kind, prec, lengths, batch, lib=lib)
            rt = torch.float32 if prec == rf.SINGLE else torch.float64
            ct = torch.complex64 if prec == rf.SINGLE else torch.complex128
            total = 1
            for v in lengths:
                total *= v
            h = total // lengths[0] * (lengths[0] // 2 + 1)
            if inplace:
                out = None
            elif kind == rf.REAL_FORWARD:
                out = torch.empty((batch, h), dtype=ct, device=dev)
            elif kind == rf.REAL_INVERSE:
                out = torch.empty((batch, total), dtype=rt, device=dev)
            else:
                out = torch.empty((batch, total), dtype=ct, device=dev)
            info = rf.ExecutionInfo(lib)
            info.set_stream(stream_ptr)
            wb = plan.work_buffer_size
            if wb:
                work = torch.empty(wb, dtype=torch.uint8, device=dev)
                info.set_work_buffer(work.data_ptr(), wb)
                self.keep.append(work)
            self.calls.append((plan, cur, out, info))
            cur = cur if inplace else out
        self.result = cur

    def run(self):
        for plan, src, dst, info in self.calls:
            plan.execute([src.data_ptr()], None if dst is None else [dst.data_ptr()], info)

    def profile(self):
        """[(pass name, bytes read+written, ms)] of one step, every kernel bracketed by events"""
        rows = []
        for plan, src, dst, info in self.calls:
            ms = plan.execute_profile([src.data_ptr()], None if dst is None else [dst.data_ptr()], info)
            for (name, nbytes), t in zip(plan.passes(), ms):
                rows.append((name, nbytes, t))
        return rows


def time_steps(torch, step, warmup, steps, settle_ms=0.0):
    """`warmup` untimed steps (and, where asked for, as many more as it takes to fill settle_ms of
    wall time: the short configurations do not reach settled clocks in 30 steps), then `steps` timed"""
    t_begin = time.perf_counter()
    for _ in range(warmup):
        step.run()
    torch.cuda.synchronize()
    while (time.perf_counter() - t_begin) * 1e3 < settle_ms:
        for _ in range(10):
            step.run()
        torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        step.run()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    dev = start.elapsed_time(stop) / steps
    # the driver checks against its own wall clock: report the larger of the two
    return max(wall, dev), dev


def kernel_profile(step, reps):
    acc = None
    for _ in range(reps):
        rows = step.profile()
        if acc is None:
            acc = [[name, nbytes, 0.0] for name, nbytes, _ in rows]
        for a, (_, _, t) in zip(acc, rows):
            a[2] += t / reps
    return acc


def cpu_port(cfg_id, wl, budget_s=6.0):
    """the CPU checker (double precision port, OpenMP over the batch) on a bounded sample"""
    import inputs
    from oracle import oracle as orc

    kinds = {0: orc.COMPLEX_FORWARD, 1: orc.COMPLEX_INVERSE, 2: orc.REAL_FORWARD, 3: orc.REAL_INVERSE}
    full_batch = wl["transforms"][0][2]
    lengths = wl["transforms"][0][1]

    def run(nb):
        x = inputs.config_input(cfg_id, 0, nb)
        t0 = time.perf_counter()
        cur = x
        for (kind, ln, _, _, _) in wl["transforms"]:
            cur = orc.transform(kinds[kind], ln, nb, cur, ld=False)
        return time.perf_counter() - t0

    threads = orc.num_threads()
    nb = min(full_batch, max(1, threads))
    t = run(nb)
    target = int(min(full_batch, max(nb, nb * budget_s / max(t, 1e-6))))
    target = max(threads, target // threads * threads) if full_batch >= threads else full_batch
    target = min(target, full_batch)
    if target > nb:
        t = run(target)
        nb = target
    frac = nb / full_batch
    return dict(value=wl["flops"] * frac / t / 1e9, unit="GFLOP/s", cores=threads, kind="port",
                sample="%d of %d transforms of %s, %.1f s, oracle/fft_oracle.c double build, %d OpenMP threads"
                % (nb, full_batch, "x".join(map(str, lengths)), t, threads))


def host_threads():
    """threads for the CPU baselines: the CPUs this process may run on (the reference's tests
    size FFTW's thread pool the same way, shared/concurrency.h:33-41), at most 16"""
    try:
        n = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        n = os.cpu_count() or 1
    return max(1, min(16, n))


def cpu_pocketfft(cfg_id, wl, budget_s=10.0, min_s=1.0):
    """scipy.fft (pocketfft, C++) on the same workload in the workload's own precision: batched
    contiguous out-of-place transforms, `workers` threads across the batch, planning (pocketfft
    caches its plans after the first call) outside the timed repetitions.  The sample is at
    least 1024 signals of the batched workloads and is repeated for at least min_s seconds."""
    import numpy as np
    import scipy.fft as sf

    import inputs

    threads = host_threads()
    full = wl["transforms"][0][2]
    lengths = wl["transforms"][0][1]
    nb = {1: 1024, 2: 1024, 3: 2, 4: 1, 5: 16}[cfg_id]
    x = inputs.config_input(cfg_id, 0, nb)
    if cfg_id in (1, 3):
        x = x.astype(np.complex64)
    elif cfg_id == 2:
        x = x.astype(np.float32)
    if cfg_id == 3:
        x = x.reshape(nb, 4096, 4096)
    elif cfg_id == 4:
        x = x.reshape(512, 512, 512)

    def run():
        if cfg_id == 2:
            return sf.irfft(sf.rfft(x, axis=1, workers=threads), n=65536, axis=1, workers=threads)
        if cfg_id == 3:
            return sf.fft2(x, axes=(1, 2), workers=threads)
        if cfg_id == 4:
            return sf.irfftn(sf.rfftn(x, workers=threads), s=(512, 512, 512), workers=threads)
        return sf.fft(x, axis=1, workers=threads)

    run()
    ts = []
    t_all = time.perf_counter()
    while (time.perf_counter() - t_all < min_s or len(ts) < 3) and time.perf_counter() - t_all < budget_s:
        t0 = time.perf_counter()
        run()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    t = ts[len(ts) // 2]
    return dict(value=wl["flops"] * (nb / full) / t / 1e9, unit="GFLOP/s", cores=threads,
                kind="library: scipy.fft (pocketfft) %s, %s" % (x.dtype, "rfft + irfft" if cfg_id in (2, 4) else "fft"),
                sample="%d of %d transforms of %s, median of %d repetitions of %.3f s (%.1f s in all), %d workers"
                % (nb, full, "x".join(map(str, lengths)), len(ts), t, sum(ts), threads))


def cpu_baseline(cfg_id, wl):
    """The fastest CPU figure this machine offers, in the order the reference's own tests would
    find one: FFTW (the reference's CPU path, clients/tests/CMakeLists.txt:128-129), MKL's FFTW
    interface, scipy's pocketfft, this repository's port.  `chain` records what each probe found;
    the others are reported under cpu_other."""
    import ctypes

    chain = {}
    for name in ("libfftw3f.so.3", "libfftw3.so.3", "libfftw3f_threads.so.3", "libfftw3f_omp.so.3", "libmkl_rt.so",
                 "libmkl_rt.so.2"):
        try:
            ctypes.CDLL(name)
            chain[name] = True
        except OSError:
            chain[name] = False
    cands = {}
    if cfg_id == 2 and chain.get("libfftw3f.so.3"):
        try:
            cands["fftw"] = fftw_r2c_c2r(wl)
        except Exception as e:  # noqa: BLE001
            cands["fftw"] = {"error": repr(e)[:200]}
    try:
        cands["pocketfft"] = cpu_pocketfft(cfg_id, wl)
    except Exception as e:  # noqa: BLE001
        cands["pocketfft"] = {"error": repr(e)[:200]}
    try:
        cands["port"] = cpu_port(cfg_id, wl)
    except Exception as e:  # noqa: BLE001
        cands["port"] = {"error": repr(e)[:200]}
    ok = {k: v for k, v in cands.items() if "value" in v}
    # FFTW when present (it is the reference's own CPU path), else the fastest of the others
    pick = "fftw" if "fftw" in ok else max(ok, key=lambda k: ok[k]["value"])
    base = dict(ok[pick])
    base["chain"] = chain
    other = {k: v for k, v in cands.items() if k != pick}
    other["dlopen"] = chain
    return base, other


def torch_fft_ms(torch, cfg_id, step, reps=5):
    """torch.fft on the same input (reference rocFFT behind hipFFT, PyTorch's output
    allocations inside the timed region); median ms per step"""
    x = step.x

    def run():
        if cfg_id == 1:
            return torch.fft.fft(x, dim=1)
        if cfg_id == 2:
            return torch.fft.irfft(torch.fft.rfft(x, dim=1), n=65536, dim=1, norm="forward")
        if cfg_id == 3:
            return torch.fft.fft2(x.reshape(8, 4096, 4096))
        if cfg_id == 4:
            return torch.fft.irfftn(torch.fft.rfftn(x.reshape(512, 512, 512)), s=(512, 512, 512), norm="forward")
        return torch.fft.fft(x, dim=1)

    try:
        run()
        torch.cuda.synchronize()
        ts = []
        for _ in range(reps):
            a = torch.cuda.Event(enable_timing=True)
            b = torch.cuda.Event(enable_timing=True)
            a.record()
            run()
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b))
        ts.sort()
        return ts[len(ts) // 2]
    except Exception:  # noqa: BLE001  (a baseline, never fatal)
        return None


def reference_library_paths():
    """copies of the reference library on this machine: the system ROCm's and the one PyTorch bundles"""
    import importlib.util

    paths = []
    for p in ("/opt/rocm/lib/librocfft.so.0",):
        if os.path.exists(p):
            paths.append(p)
    spec = importlib.util.find_spec("torch")
    if spec and spec.origin:
        p = os.path.join(os.path.dirname(spec.origin), "lib", "librocfft.so")
        if os.path.exists(p):
            paths.append(p)
    return paths


def reference_child(path, warmup, steps):
    """(child process) the five configurations on the library at `path` through the same Step
    harness as this library; prints one JSON line {"version": ..., "ms": {name: ms}}"""
    import torch

    import rocfft_amd.binding as B

    lib = B.Library(path, extensions=False)
    lib.setup()
    out = {"path": path, "version": lib.version(), "ms": {}, "steps": steps, "warmup": warmup}
    stream_ptr = torch.cuda.current_stream().cuda_stream
    wls = workloads()
    for cid in sorted(wls):
        try:
            step = Step(cid, wls[cid], torch, stream_ptr, lib=lib)
            ms, _ = time_steps(torch, step, warmup, steps, EXTRA_SETTLE_MS)
            out["ms"][wls[cid]["name"]] = ms
            del step
            torch.cuda.empty_cache()
        except Exception as e:  # noqa: BLE001
            out["ms"][wls[cid]["name"]] = None
            out.setdefault("errors", {})[wls[cid]["name"]] = repr(e)[:200]
    print(json.dumps(out))


def reference_rocfft(warmup, steps, timeout_s=240):
    """runs reference_child once per copy of the reference library, each in its own process
    (a library that cannot share this process's HIP runtime must not take the benchmark down)"""
    import subprocess

    results = []
    for path in reference_library_paths():
        rec = {"path": path, "version": None, "ms": {}}
        try:
            p = subprocess.run([sys.executable, os.path.abspath(__file__), "--reference-lib", path, "--steps",
                                str(steps), "--warmup", str(warmup)], capture_output=True, text=True,
                               timeout=timeout_s)
            line = [ln for ln in p.stdout.strip().splitlines() if ln.startswith("{")]
            if p.returncode == 0 and line:
                rec = json.loads(line[-1])
            else:
                rec["error"] = ("exit %d: " % p.returncode) + p.stderr.strip()[-200:]
        except Exception as e:  # noqa: BLE001
            rec["error"] = repr(e)[:200]
        results.append(rec)
    return results


def fftw_r2c_c2r(wl, budget_s=10.0, min_s=1.0):
    """FFTW single precision, batched contiguous out-of-place plans with FFTW_ESTIMATE as the
    reference's tests make them (shared/rocfft_against_fftw.h:108-142); one thread unless the
    threads library is present"""
    import ctypes

    import numpy as np

    import inputs

    n, full, nb = 65536, 4096, 1024
    x = inputs.config_input(2, 0, nb).astype(np.float32)
    fw = ctypes.CDLL("libfftw3f.so.3")
    threads = 1
    for tl in ("libfftw3f_omp.so.3", "libfftw3f_threads.so.3"):
        try:
            ft = ctypes.CDLL(tl, mode=ctypes.RTLD_GLOBAL)
            ft.fftwf_init_threads()
            threads = host_threads()
            ft.fftwf_plan_with_nthreads(threads)
            break
        except (OSError, AttributeError):
            continue
    h = n // 2 + 1
    y = np.empty((nb, h), dtype=np.complex64)
    z = np.empty((nb, n), dtype=np.float32)
    nn = (ctypes.c_int * 1)(n)
    fw.fftwf_plan_many_dft_r2c.restype = ctypes.c_void_p
    fw.fftwf_plan_many_dft_c2r.restype = ctypes.c_void_p
    FFTW_ESTIMATE = 1 << 6
    pf = fw.fftwf_plan_many_dft_r2c(1, nn, nb, ctypes.c_void_p(x.ctypes.data), None, 1, n,
                                    ctypes.c_void_p(y.ctypes.data), None, 1, h, FFTW_ESTIMATE)
    pb = fw.fftwf_plan_many_dft_c2r(1, nn, nb, ctypes.c_void_p(y.ctypes.data), None, 1, h,
                                    ctypes.c_void_p(z.ctypes.data), None, 1, n, FFTW_ESTIMATE)
    if not pf or not pb:
        raise RuntimeError("fftwf_plan_many_dft failed")
    fw.fftwf_execute.argtypes = [ctypes.c_void_p]
    ts = []
    t_all = time.perf_counter()
    while (time.perf_counter() - t_all < min_s or len(ts) < 3) and time.perf_counter() - t_all < budget_s:
        t0 = time.perf_counter()
        fw.fftwf_execute(pf)
        fw.fftwf_execute(pb)
        ts.append(time.perf_counter() - t0)
    ts.sort()
    t = ts[len(ts) // 2]
    return dict(value=wl["flops"] * (nb / full) / t / 1e9, unit="GFLOP/s", cores=threads,
                kind="reference: FFTW 3 float32, FFTW_ESTIMATE",
                sample="%d of %d transforms of %d, median of %d repetitions of %.3f s" % (nb, full, n, len(ts), t))


def copy_probes():
    """name -> fields of rocfft_amd_copy_probe: plain copies of 1 GiB in the access shapes of the
    passes of the five configurations (element = 8 bytes unless said)"""
    import rocfft_amd.binding as B

    gib = 1 << 30
    rows = 4096  # rows of 32768 elements of 8 bytes: 1 GiB
    tiles = dict(shape=B.PROBE_TILES, rows=0, tile_width=64, elem_bytes=8)
    return {
        "stream, 16 B per lane, 4 workgroups per CU": dict(shape=B.PROBE_STREAM, bytes=gib),
        "stream, nontemporal": dict(shape=B.PROBE_STREAM, bytes=gib, nontemporal=1),
        "stream, 8 workgroups per CU": dict(shape=B.PROBE_STREAM, bytes=gib, workgroups_per_cu=8),
        "stream, 64 workgroups per CU": dict(shape=B.PROBE_STREAM, bytes=gib, workgroups_per_cu=64),
        "read only": dict(shape=B.PROBE_READ, bytes=gib),
        "write only": dict(shape=B.PROBE_WRITE, bytes=gib),
        # configuration 2: one workgroup of 1024 threads per row of 256 KiB
        "rows of 32768, 32 loads then 32 stores, 1 workgroup per CU": dict(shape=B.PROBE_ROWS, rows=rows, in_row=32768, out_row=32768, group=32, workgroups_per_cu=1),
        "rows of 32768, 8 loads then 8 stores, 1 workgroup per CU": dict(shape=B.PROBE_ROWS, rows=rows, in_row=32768, out_row=32768, group=8, workgroups_per_cu=1),
        "rows of 32768, 4 loads then 4 stores, 1 workgroup per CU": dict(shape=B.PROBE_ROWS, rows=rows, in_row=32768, out_row=32768, group=4, workgroups_per_cu=1),
        "rows of 32768, 2 loads then 2 stores, 1 workgroup per CU": dict(shape=B.PROBE_ROWS, rows=rows, in_row=32768, out_row=32768, group=2, workgroups_per_cu=1),
        "rows of 32768, 1 load then 1 store, 1 workgroup per CU": dict(shape=B.PROBE_ROWS, rows=rows, in_row=32768, out_row=32768, group=1, workgroups_per_cu=1),
        "rows of 32768 read, rows 32769 apart written (real forward), 32/32": dict(shape=B.PROBE_ROWS, rows=rows, in_row=32768, out_row=32769, group=32, workgroups_per_cu=1),
        "rows 32769 apart read, rows of 32768 written (real inverse), 32/32": dict(shape=B.PROBE_ROWS, rows=rows, in_row=32769, out_row=32768, group=32, workgroups_per_cu=1),
        "rows 32769 apart written, 8/8": dict(shape=B.PROBE_ROWS, rows=rows, in_row=32768, out_row=32769, group=8, workgroups_per_cu=1),
        "rows 32769 apart written, 32/32, 2 workgroups per CU": dict(shape=B.PROBE_ROWS, rows=rows, in_row=32768, out_row=32769, group=32, workgroups_per_cu=2),
        # configurations 1 and 3, row pass: a tile is one contiguous row of 4096 elements
        "tiles 4096 x 1 (contiguous rows of 32 KiB), one workgroup per tile": dict(tiles, tile_width=256, in_row=256, out_row=256, tiles_per_slab=1, rows=32768, in_slab=4096, out_slab=4096),
        "tiles 4096 x 1, nontemporal": dict(tiles, tile_width=256, in_row=256, out_row=256, tiles_per_slab=1, rows=32768, in_slab=4096, out_slab=4096, nontemporal=1),
        "tiles 4096 x 1, resident grid": dict(tiles, tile_width=256, in_row=256, out_row=256, tiles_per_slab=1, rows=32768, in_slab=4096, out_slab=4096, resident_grid=1),
        # configuration 3, column passes over 8 arrays of 4096 rows of 4096 elements: a tile is 64
        # columns x 64 rows, the rows adjacent (first pass of the split) or 64 rows apart (second pass)
        "tiles 64 x 64, adjacent rows of 4096 (configuration 3, first column pass)": dict(tiles, in_row=4096, out_row=4096, tiles_per_slab=64, rows=512, in_slab=64 * 4096, out_slab=64 * 4096),
        "tiles 64 x 64, adjacent rows of 4096, nontemporal": dict(tiles, in_row=4096, out_row=4096, tiles_per_slab=64, rows=512, in_slab=64 * 4096, out_slab=64 * 4096, nontemporal=1),
        "tiles 64 x 64, adjacent rows of 4096, resident grid": dict(tiles, in_row=4096, out_row=4096, tiles_per_slab=64, rows=512, in_slab=64 * 4096, out_slab=64 * 4096, resident_grid=1),
        "tiles 64 x 64, rows 64 x 4096 apart (configuration 3, second column pass)": dict(tiles, in_row=64 * 4096, out_row=64 * 4096, tiles_per_slab=64, rows=512, in_slab=4096, out_slab=4096, slabs_inner=64, in_slab_outer=4096 * 4096, out_slab_outer=4096 * 4096),
        "tiles 64 x 64, rows 64 x 4096 apart, nontemporal": dict(tiles, in_row=64 * 4096, out_row=64 * 4096, tiles_per_slab=64, rows=512, in_slab=4096, out_slab=4096, slabs_inner=64, in_slab_outer=4096 * 4096, out_slab_outer=4096 * 4096, nontemporal=1),
        "tiles 64 x 64, adjacent rows 4096 + 32 apart (256 bytes of padding)": dict(tiles, in_row=4128, out_row=4128, tiles_per_slab=64, rows=512, in_slab=64 * 4128, out_slab=64 * 4128),
        "tiles 64 x 64, adjacent rows 4096 + 64 apart (512 bytes of padding)": dict(tiles, in_row=4160, out_row=4160, tiles_per_slab=64, rows=512, in_slab=64 * 4160, out_slab=64 * 4160),
        # configuration 4, column passes: 8 columns of 16 bytes x 512 rows
        "tiles 8 x 512 of 16 B, rows 257 apart, each XCD a range of tiles (configuration 4, y columns)": dict(tiles, tile_width=8, elem_bytes=16, in_row=257, out_row=257, tiles_per_slab=32, rows=512, in_slab=257 * 512, out_slab=257 * 512, xcd_ranges=1),
        "tiles 8 x 512 of 16 B, rows 257 apart, workgroups round-robin over the XCDs": dict(tiles, tile_width=8, elem_bytes=16, in_row=257, out_row=257, tiles_per_slab=32, rows=512, in_slab=257 * 512, out_slab=257 * 512),
        "tiles 8 x 512 of 16 B, rows 131584 apart (configuration 4, z columns)": dict(tiles, tile_width=8, elem_bytes=16, in_row=131584, out_row=131584, tiles_per_slab=16384, rows=1, in_slab=0, out_slab=0),
        "tiles 8 x 512 of 16 B, rows 131584 apart, nontemporal": dict(tiles, tile_width=8, elem_bytes=16, in_row=131584, out_row=131584, tiles_per_slab=16384, rows=1, in_slab=0, out_slab=0, nontemporal=1),
        "tiles 16 x 256 of 16 B, rows 131584 apart": dict(tiles, tile_width=16, elem_bytes=16, in_row=131584, out_row=131584, tiles_per_slab=8192, rows=2, in_slab=131584 * 256, out_slab=131584 * 256),
    }


def copy_ceilings(torch, lib, names=None, reps=10):
    """name -> (median ms, TB/s counting bytes read + bytes written) of the copy probes"""
    import rocfft_amd.binding as B

    dev = torch.device("cuda:0")
    src = torch.rand((1 << 28) + (1 << 22), dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    stream_ptr = torch.cuda.current_stream().cuda_stream
    out = {}
    for name, f in copy_probes().items():
        if names is not None and name not in names:
            continue
        f = dict(f, src=src.data_ptr(), dst=dst.data_ptr())
        if f["shape"] == B.PROBE_ROWS:
            moved = 2.0 * f["rows"] * 32768 * 8
        elif f["shape"] == B.PROBE_TILES:
            moved = 2.0 * f["tiles_per_slab"] * f["rows"] * 4096 * f["elem_bytes"]
        elif f["shape"] == B.PROBE_STREAM:
            moved = 2.0 * f["bytes"]
        else:
            moved = 1.0 * f["bytes"]
        # (enough launches for the clocks to settle, as the warm-up steps of the benchmark)
        for _ in range(60):
            lib.copy_probe(stream_ptr, **f)
        torch.cuda.synchronize()
        ts = []
        for _ in range(reps):
            a = torch.cuda.Event(enable_timing=True)
            b = torch.cuda.Event(enable_timing=True)
            a.record()
            lib.copy_probe(stream_ptr, **f)
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b))
        ts.sort()
        ms = ts[len(ts) // 2]
        out[name] = (ms, moved / (ms * 1e-3) / 1e12)
    return out


# the copy probe whose access shape is that of the slowest kernel of a configuration
SHAPE_OF_CONFIG = {
    1: "tiles 4096 x 1 (contiguous rows of 32 KiB), one workgroup per tile",
    2: "rows 32769 apart read, rows of 32768 written (real inverse), 32/32",
    3: "tiles 64 x 64, rows 64 x 4096 apart (configuration 3, second column pass)",
    4: "tiles 8 x 512 of 16 B, rows 131584 apart (configuration 4, z columns)",
    5: "tiles 4096 x 1 (contiguous rows of 32 KiB), one workgroup per tile",
}


# warm-up and timed steps of the other configurations and of the reference library; their warm-up
# lasts 30 ms at least (30 steps of configuration 1 are 0.5 ms)
EXTRA_WARMUP, EXTRA_STEPS, EXTRA_SETTLE_MS = 30, 20, 30.0


def measure_config(torch, cfg_id, wl, stream_ptr, warmup, steps, prof_reps, settle_ms=0.0):
    step = Step(cfg_id, wl, torch, stream_ptr)
    ms, dev_ms = time_steps(torch, step, warmup, steps, settle_ms)
    prof = kernel_profile(step, prof_reps)
    return step, ms, dev_ms, prof


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    # The clocks of the part settle during the first 25-30 ms of back-to-back launches (the kernels of
    # configuration 2 take 0.49 / 0.51 ms at first, up to 0.57 ms after 3-7 ms and 0.47 / 0.49 ms from
    # 25 ms on): the default warm-up covers that, and the other configurations and the reference
    # library are timed after the same number of warm-up steps.
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1..5 (default 2)")
    ap.add_argument("--no-extras", action="store_true", help="skip all_configs and the CPU baseline")
    ap.add_argument("--reference-lib", default=None,
                    help="(used by this script for its child processes) time the five configurations on the "
                         "rocfft.h library at this path and print them as JSON")
    ap.add_argument("--copy-ceilings", action="store_true",
                    help="time plain copies of 1 GiB in the access shapes of the passes (rocfft_amd_copy_probe) and "
                         "print them as a table: what the memory system gives a copy of each shape")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain elementwise copy of 1 GiB (reads 1 GiB, writes 1 GiB) ten times: "
                         "the known-size kernel the rocprofv3 FETCH_SIZE/WRITE_SIZE counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build drives one GPU; --gpus %d is not supported "
              "(every transform of these workloads shards by batch without communication)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    # the reference library's figures come from child processes, started before this process
    # initialises the GPU
    refs = []
    if not (args.no_extras or args.reference_lib or args.calibrate_copy or args.copy_ceilings):
        refs = reference_rocfft(EXTRA_WARMUP, EXTRA_STEPS)

    import torch

    import rocfft_amd as rf

    if not torch.cuda.is_available():
        print("bench.py: no GPU", file=sys.stderr)
        sys.exit(1)
    if args.reference_lib:
        reference_child(args.reference_lib, args.warmup, args.steps)
        return
    if args.calibrate_copy:
        n = 1 << 28  # float32 elements = 1 GiB
        src = torch.rand(n, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(10):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "torch.mul(src, 1.0, out=dst), float32", "bytes_read": 4 * n,
                          "bytes_written": 4 * n, "launches": 10}))
        return
    lib = rf.library()  # raises if the HIP library is not built
    if args.copy_ceilings:
        res = copy_ceilings(torch, lib)
        print("| copy of 1 GiB (1 GiB read, 1 GiB written unless said) | ms | TB/s | of 8 TB/s |")
        print("|---|---|---|---|")
        for name, (ms, tbs) in res.items():
            print("| %s | %.3f | %.2f | %.3f |" % (name, ms, tbs, tbs * 1e3 / HBM_PEAK_GBS))
        print(json.dumps({"copy_ceilings_TBps": {k: v[1] for k, v in res.items()}}))
        return
    stream_ptr = torch.cuda.current_stream().cuda_stream
    wls = workloads()
    wl = wls[args.config]

    step, ms, dev_ms, prof = measure_config(torch, args.config, wl, stream_ptr, args.warmup, args.steps, 5)
    dom = max(prof, key=lambda r: r[2])
    achieved = dom[1] / (dom[2] * 1e-3) / 1e9
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        try:
            traffic = json.load(open(tpath)).get(wl["name"], {}).get(dom[0])
        except Exception:  # noqa: BLE001
            traffic = None
    # the same kernel against a plain copy in its access shape, and against the best copy seen
    shape = SHAPE_OF_CONFIG[args.config]
    best = "stream, nontemporal"
    try:
        cc = copy_ceilings(torch, lib, names={shape, best})
        copy_shape, copy_best = cc[shape][1] * 1e3, cc[best][1] * 1e3
    except Exception:  # noqa: BLE001
        copy_shape = copy_best = None
    out = {
        "metric": "GFLOP/s (5N*log2N) per config, 1 GPU",
        "value": wl["flops"] / (ms * 1e-3) / 1e9,
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": wl["dtype"],
        "data": "synthetic",
        "config": {"workload": wl["name"], "transforms_per_step": len(wl["transforms"]),
                   "kernels_per_step": len(prof)},
        "device_ms_per_step": dev_ms,
        "algorithmic_GBps": wl["bytes"] / (ms * 1e-3) / 1e9,
        "algorithmic_hbm_frac": wl["bytes"] / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "kernel": dom[0],
                     "kernel_ms": dom[2], "kernel_bytes": dom[1],
                     "frac_of_copy": achieved / copy_shape if copy_shape else None,
                     "copy_of_shape_GBps": copy_shape, "copy_shape": shape,
                     "best_copy_GBps": copy_best},
        "kernels": [{"name": n, "bytes": b, "ms": t, "GBps": b / (t * 1e-3) / 1e9 if t > 0 else None}
                    for n, b, t in prof],
    }
    if not args.no_extras:
        tf_ms = torch_fft_ms(torch, args.config, step)
        allc = {}
        for cid in sorted(wls):
            if cid == args.config:
                s2, m2, p2 = step, ms, prof
                t2 = tf_ms
            else:
                del step
                torch.cuda.empty_cache()
                s2, m2, _, p2 = measure_config(torch, cid, wls[cid], stream_ptr, EXTRA_WARMUP, EXTRA_STEPS, 2, EXTRA_SETTLE_MS)
                t2 = torch_fft_ms(torch, cid, s2)
                step = s2
            w2 = wls[cid]
            # reference rocFFT through the identical harness: the fastest copy found on this machine
            same = [(r["ms"].get(w2["name"]), r.get("version"), r.get("path")) for r in refs
                    if r.get("ms", {}).get(w2["name"])]
            r2 = min(same) if same else (None, None, None)
            allc[w2["name"]] = {
                "ms": m2, "GFLOPs": w2["flops"] / (m2 * 1e-3) / 1e9,
                "GBps": w2["bytes"] / (m2 * 1e-3) / 1e9,
                "hbm_frac": w2["bytes"] / (m2 * 1e-3) / 1e9 / HBM_PEAK_GBS,
                "kernels": len(p2),
                "reference_rocfft_ms": r2[0],
                "reference_rocfft_version": r2[1],
                "reference_rocfft_GFLOPs": (w2["flops"] / (r2[0] * 1e-3) / 1e9) if r2[0] else None,
                "torch_fft_ms": t2,
            }
        out["all_configs"] = allc
        out["reference_rocfft"] = refs
        del step
        torch.cuda.empty_cache()
        out["cpu_baseline"], out["cpu_other"] = cpu_baseline(args.config, wl)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
