"""Command-line benchmark with the options and output of the reference's rocfft-bench.

    python -m rocfft_amd.bench_cli --token complex_forward_len_4096_single_ip_batch_1024_istride_1_CI_ostride_1_CI_idist_4096_odist_4096_ioffset_0_0_ooffset_0_0 -N 10
    python -m rocfft_amd.bench_cli --length 512 512 512 -t 2 --precision double -o -N 5

Option names, the trial loop (one warm-up execute, then N executes each bracketed by two
events on the execution stream) and the two result lines ("Execution gpu time", "Execution
gflops") follow clients/bench/bench.cpp:60-140, :383-480 of the reference, so scripts that
parse rocfft-bench's output read this one too.  Lengths and strides are row-major, as there.
Device buffers come from torch; everything timed is `rocfft_execute` of this library.
"""
import argparse
import sys

from . import binding as B
from .params import FFTParams, TokenError

_ARRAY_TYPES = {"0": B.COMPLEX_INTERLEAVED, "1": B.COMPLEX_PLANAR, "2": B.REAL, "3": B.HERMITIAN_INTERLEAVED,
                "4": B.HERMITIAN_PLANAR}


def parse(argv):
    ap = argparse.ArgumentParser(prog="rocfft_amd.bench_cli", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--version", action="store_true", help="print the library version string")
    ap.add_argument("--token", default="", help="token to read the transform parameters from")
    ap.add_argument("-t", "--transformType", type=int, default=0,
                    help="0 complex forward, 1 complex inverse, 2 real forward, 3 real inverse")
    ap.add_argument("--precision", default="single", choices=["single", "double", "half"])
    ap.add_argument("--double", action="store_true", help="deprecated: use --precision double")
    ap.add_argument("-o", "--notInPlace", action="store_true", help="not in-place (default: in-place)")
    ap.add_argument("--itype", default=None, choices=list(_ARRAY_TYPES), help="array type of the input")
    ap.add_argument("--otype", default=None, choices=list(_ARRAY_TYPES), help="array type of the output")
    ap.add_argument("--length", type=int, nargs="+", default=[], help="1 to 3 lengths, slowest first")
    ap.add_argument("-b", "--batchSize", type=int, default=1)
    ap.add_argument("--istride", type=int, nargs="+", default=[])
    ap.add_argument("--ostride", type=int, nargs="+", default=[])
    ap.add_argument("--idist", type=int, default=0)
    ap.add_argument("--odist", type=int, default=0)
    ap.add_argument("--ioffset", type=int, nargs="+", default=[])
    ap.add_argument("--ooffset", type=int, nargs="+", default=[])
    ap.add_argument("--scalefactor", type=float, default=1.0)
    ap.add_argument("-N", "--ntrial", type=int, default=1)
    ap.add_argument("--device", type=int, default=0)
    ap.add_argument("--verbose", type=int, default=0)
    return ap.parse_args(argv)


def params_from_args(a):
    if a.token:
        return FFTParams.from_token(a.token)
    if not a.length:
        raise TokenError("--length or --token is needed")
    prec = B.DOUBLE if (a.double or a.precision == "double") else B.HALF if a.precision == "half" else B.SINGLE
    return FFTParams(a.transformType, a.length, prec, B.NOTINPLACE if a.notInPlace else B.INPLACE, a.batchSize,
                     a.istride, a.ostride, a.idist, a.odist, a.ioffset, a.ooffset,
                     _ARRAY_TYPES[a.itype] if a.itype else None, _ARRAY_TYPES[a.otype] if a.otype else None,
                     a.scalefactor)


def main(argv=None):
    a = parse(sys.argv[1:] if argv is None else argv)
    import torch  # before the library: both must share one HIP runtime

    lib = B.library()
    if a.version:
        print("version", lib.version())
        return 0
    try:
        p = params_from_args(a).validate()
    except TokenError as e:
        print("error:", e, file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("error: no GPU", file=sys.stderr)
        return 1
    torch.cuda.set_device(a.device)
    dev = torch.device("cuda", a.device)
    print("Token:", p.token())
    plan = p.make_plan(lib)
    if a.verbose:
        plan.print()

    scalar = torch.float64 if p.precision == B.DOUBLE else torch.float32
    per_in = 1 if p.itype == B.REAL or p.ibuffers() == 2 else 2   # scalars per element and buffer
    per_out = 1 if p.otype == B.REAL or p.obuffers() == 2 else 2
    ibufs = [torch.rand(p.isize() * per_in, dtype=scalar, device=dev) - 0.5 for _ in range(p.ibuffers())]
    inplace = p.placement == B.INPLACE
    if inplace:
        need = max(p.isize() * per_in, p.osize() * per_out)
        if need > ibufs[0].numel():
            ibufs = [torch.rand(need, dtype=scalar, device=dev) - 0.5 for _ in range(max(p.ibuffers(), p.obuffers()))]
        obufs = None
    else:
        obufs = [torch.empty(p.osize() * per_out, dtype=scalar, device=dev) for _ in range(p.obuffers())]
    info = B.ExecutionInfo(lib)
    info.set_stream(torch.cuda.current_stream().cuda_stream)
    wb = plan.work_buffer_size
    work = None
    if wb:
        work = torch.empty(wb, dtype=torch.uint8, device=dev)
        info.set_work_buffer(work.data_ptr(), wb)
    iptrs = [t.data_ptr() for t in ibufs]
    optrs = None if obufs is None else [t.data_ptr() for t in obufs]

    plan.execute(iptrs, optrs, info)  # warm-up
    torch.cuda.synchronize()
    times = []
    for _ in range(max(1, a.ntrial)):
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        plan.execute(iptrs, optrs, info)
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop))
    print("\nExecution gpu time:" + "".join(" %g" % t for t in times) + " ms")
    ops = p.opscount()
    print("Execution gflops:  " + "".join(" %g" % (ops / (1e6 * t)) for t in times))
    return 0


if __name__ == "__main__":
    sys.exit(main())
