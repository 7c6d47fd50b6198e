"""Seeded, counter-based synthetic inputs shared by every implementation under
test (the CPU checker, the GPU library, numpy when the fixtures are written).

value(seed, i) depends only on (seed, i), so any slice of a large input can be
produced without generating the rest, and the bytes do not depend on the numpy
version.  splitmix64 finaliser -> 53 random bits -> uniform double in [0, 1).
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix(z):
    z = np.asarray(z, dtype=np.uint64).reshape(-1) if np.isscalar(z) or np.ndim(z) == 0 else z
    z = (z + np.uint64(0x9E3779B97F4A7C15)) & _M64
    z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
    z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
    return z ^ (z >> np.uint64(31))


def uniform01(seed, start, count):
    """count doubles in [0,1): elements start .. start+count-1 of stream `seed`."""
    with np.errstate(over="ignore"):
        idx = np.arange(start, start + count, dtype=np.uint64)
        z = _splitmix(idx ^ _splitmix(np.uint64(seed))[0])
    return (z >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def real_input(seed, start, count):
    """reals i.i.d. uniform in [-1, 1) (the real-transform configs)."""
    return uniform01(seed, start, count) * 2.0 - 1.0


def complex_input(seed, start, count):
    """complex values, re and im i.i.d. uniform in [-0.5, 0.5) (the complex configs);
    element k uses stream positions 2k and 2k+1."""
    u = uniform01(seed, 2 * start, 2 * count) - 0.5
    return u.view(np.complex128)


# The five benchmark configurations (lengths fastest-first as in rocfft.h).
CONFIGS = {
    1: dict(kind="c2c", lengths=[4096], batch=1024, precision="single", placement="inplace", seed=101),
    2: dict(kind="r2c", lengths=[65536], batch=4096, precision="single", placement="notinplace", seed=102),
    3: dict(kind="c2c", lengths=[4096, 4096], batch=8, precision="single", placement="notinplace", seed=103),
    4: dict(kind="r2c", lengths=[512, 512, 512], batch=1, precision="double", placement="notinplace", seed=104),
    5: dict(kind="c2c", lengths=[1000003], batch=16, precision="double", placement="notinplace", seed=105),
}


def config_input(cfg_id, first_batch=0, nbatch=None):
    """Input of batches [first_batch, first_batch+nbatch) of a configuration, float64/complex128,
    shape (nbatch, prod(lengths))."""
    c = CONFIGS[cfg_id]
    total = int(np.prod(c["lengths"]))
    nbatch = c["batch"] if nbatch is None else nbatch
    if c["kind"] == "c2c":
        x = complex_input(c["seed"], first_batch * total, nbatch * total)
    else:
        x = real_input(c["seed"], first_batch * total, nbatch * total)
    return x.reshape(nbatch, total)


def sample_bins(cfg_id, count=96):
    """Deterministic output positions (flat indices into one transform's output) kept in the
    golden fixtures: the first and last 8 plus pseudo-random ones."""
    c = CONFIGS[cfg_id]
    lengths = list(c["lengths"])
    if c["kind"] == "r2c":
        lengths[0] = lengths[0] // 2 + 1
    total = int(np.prod(lengths))
    r = (uniform01(9000 + cfg_id, 0, count) * total).astype(np.int64)
    idx = np.concatenate([np.arange(8), np.arange(total - 8, total), r])
    return np.unique(idx % total)


# ---------------------------------------------------------------------------
# the same streams generated on a torch device (for the full-size GPU tests)

def _t_lsr(torch, z, k):
    """logical right shift of int64 tensors (torch's >> is arithmetic)"""
    return (z >> k) & ((1 << (64 - k)) - 1)


def _t_splitmix(torch, z):
    def c(v):  # 64-bit constant as a signed python int
        return v - (1 << 64) if v >= (1 << 63) else v

    z = z + c(0x9E3779B97F4A7C15)
    z = (z ^ _t_lsr(torch, z, 30)) * c(0xBF58476D1CE4E5B9)
    z = (z ^ _t_lsr(torch, z, 27)) * c(0x94D049BB133111EB)
    return z ^ _t_lsr(torch, z, 31)


def torch_uniform01(torch, device, seed, start, count, chunk=1 << 26):
    out = torch.empty(count, dtype=torch.float64, device=device)
    with np.errstate(over="ignore"):
        s = int(_splitmix(np.uint64(seed))[0])
    s = s - (1 << 64) if s >= (1 << 63) else s
    for lo in range(0, count, chunk):
        n = min(chunk, count - lo)
        idx = torch.arange(start + lo, start + lo + n, dtype=torch.int64, device=device)
        z = _t_splitmix(torch, idx ^ s)
        out[lo:lo + n] = _t_lsr(torch, z, 11).to(torch.float64) * (1.0 / 9007199254740992.0)
    return out


def torch_config_input(torch, device, cfg_id):
    """whole input of a configuration on `device`, in the configuration's precision"""
    c = CONFIGS[cfg_id]
    total = int(np.prod(c["lengths"]))
    single = c["precision"] == "single"
    if c["kind"] == "c2c":
        u = torch_uniform01(torch, device, c["seed"], 0, 2 * total * c["batch"]) - 0.5
        u = u.to(torch.float32) if single else u
        return torch.view_as_complex(u.reshape(c["batch"], total, 2))
    u = torch_uniform01(torch, device, c["seed"], 0, total * c["batch"]) * 2.0 - 1.0
    u = u.to(torch.float32) if single else u
    return u.reshape(c["batch"], total)
