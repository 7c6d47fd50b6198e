"""Writes the golden fixtures tests/golden/cfg<N>.npz.

Expected values come from numpy's pocketfft in float64 -- an implementation that
shares no code with the CPU checker under oracle/ or with the GPU library -- on
the seeded inputs of tests/inputs.py.  For each benchmark configuration the
fixture keeps, for the first transforms of the batch: the output at a fixed set
of positions (inputs.sample_bins), the sum of all outputs and their L2 norm.
The reference's own tests hold no stored vectors for this path (every check
there is a live FFTW comparison, shared/accuracy_test.h:881-1631), so these
fixtures are this repository's pinned known-answer data.

Run:  python tests/golden/make_golden.py   (a few minutes, ~6 GiB of memory)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import inputs  # noqa: E402

ROWS = {1: 4, 2: 2, 3: 1, 4: 1, 5: 2}


def forward(cfg_id, x):
    c = inputs.CONFIGS[cfg_id]
    shape = tuple(reversed(c["lengths"]))
    a = x.reshape((x.shape[0],) + shape)
    axes = tuple(range(1, len(shape) + 1))
    if c["kind"] == "c2c":
        y = np.fft.fftn(a, axes=axes)
    else:
        y = np.fft.rfftn(a, axes=axes)
    return y.reshape(x.shape[0], -1)


def main():
    for cfg_id in sorted(inputs.CONFIGS):
        rows = ROWS[cfg_id]
        x = inputs.config_input(cfg_id, 0, rows)
        y = forward(cfg_id, x)
        bins = inputs.sample_bins(cfg_id)
        out = dict(
            rows=np.int64(rows),
            bins=bins,
            values=y[:, bins].astype(np.complex128),
            total=y.sum(axis=1).astype(np.complex128),
            l2=np.sqrt((np.abs(y) ** 2).sum(axis=1)),
            input_head=x[:, :4].copy(),
        )
        path = os.path.join(HERE, "cfg%d.npz" % cfg_id)
        np.savez(path, **out)
        print("wrote", path, y.shape, flush=True)


if __name__ == "__main__":
    main()
