"""Child process of test_gpu_toggles.py: runs a fixed list of transforms through the library and
prints one SHA-256 per result.  The parent compares the lists of runs with different switches in
the environment (the switches are read once, when the library is loaded)."""
import hashlib
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import torch  # noqa: E402

import rocfft_amd.binding as B  # noqa: E402


def main():
    lib = B.library()
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    cases = [(B.COMPLEX_FORWARD, B.SINGLE, [4096], 64, False), (B.COMPLEX_INVERSE, B.DOUBLE, [1000], 50, True),
             (B.COMPLEX_FORWARD, B.SINGLE, [65536], 8, False), (B.REAL_FORWARD, B.SINGLE, [2048], 100, False),
             (B.REAL_INVERSE, B.SINGLE, [2048], 100, False), (B.COMPLEX_FORWARD, B.SINGLE, [64, 4096], 4, False),
             (B.COMPLEX_FORWARD, B.SINGLE, [4, 5], 3000, False), (B.REAL_FORWARD, B.DOUBLE, [6, 10], 999, False),
             (B.COMPLEX_FORWARD, B.HALF, [4096], 64, False), (B.REAL_FORWARD, B.HALF, [512, 64], 5, False),
             (B.REAL_INVERSE, B.HALF, [1024], 300, False), (B.COMPLEX_INVERSE, B.HALF, [100, 60], 9, True)]
    for kind, prec, lengths, batch, inplace in cases:
        gen.manual_seed(7)
        total = int(np.prod(lengths))
        h = total // lengths[0] * (lengths[0] // 2 + 1)
        rt = {B.SINGLE: torch.float32, B.DOUBLE: torch.float64, B.HALF: torch.float16}[prec]
        n_in = 2 * total if kind in (B.COMPLEX_FORWARD, B.COMPLEX_INVERSE) else total if kind == B.REAL_FORWARD else 2 * h
        n_out = 2 * total if kind in (B.COMPLEX_FORWARD, B.COMPLEX_INVERSE) else 2 * h if kind == B.REAL_FORWARD else total
        x = (torch.rand(batch * n_in, dtype=torch.float32, device=dev, generator=gen) - 0.5).to(rt)
        y = x if inplace else torch.zeros(batch * n_out, dtype=rt, device=dev)
        plan = B.Plan(B.INPLACE if inplace else B.NOTINPLACE, kind, prec, lengths, batch, lib=lib)
        plan.execute([x.data_ptr()], None if inplace else [y.data_ptr()])
        torch.cuda.synchronize()
        print(hashlib.sha256(y.cpu().numpy().tobytes()).hexdigest(), flush=True)
        plan.destroy()


if __name__ == "__main__":
    main()
