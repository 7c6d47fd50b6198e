"""rocfft_amd_copy_probe (include/rocfft_amd.h): the plain copies that bench.py prices the kernels
against.  Every shape has to move exactly the elements it claims to move (a probe that skipped or
doubled part of its array would report a wrong ceiling), and bad arguments are refused."""
import pytest

import rocfft_amd.binding as B


def test_probe_is_refused_without_a_gpu(emu):
    # the host emulation of the runtime layer has no probe kernels
    with pytest.raises(B.RocfftError):
        emu.copy_probe(None, shape=B.PROBE_STREAM, src=0, dst=0, bytes=16)


@pytest.mark.gpu
def test_probe_shapes_copy_what_they_claim(gpu_lib):
    import torch

    lib = gpu_lib
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    n = 1 << 21  # floats; eight rows of 32769 elements of 8 bytes fit
    src = torch.rand(n, dtype=torch.float32, device=dev)

    def fresh():
        return torch.full_like(src, -1.0)

    # stream: the first MiB, nothing beyond
    dst = fresh()
    lib.copy_probe(stream, shape=B.PROBE_STREAM, src=src.data_ptr(), dst=dst.data_ptr(), bytes=1 << 20)
    torch.cuda.synchronize()
    assert torch.equal(dst[: 1 << 18], src[: 1 << 18]) and (dst[1 << 18:] == -1).all()
    for nt in (0, 1):
        dst = fresh()
        lib.copy_probe(stream, shape=B.PROBE_STREAM, src=src.data_ptr(), dst=dst.data_ptr(), bytes=1 << 20,
                       nontemporal=nt, workgroups_per_cu=8)
        torch.cuda.synchronize()
        assert torch.equal(dst[: 1 << 18], src[: 1 << 18])

    # write only: the pattern 1, 2, 3, 4
    dst = fresh()
    lib.copy_probe(stream, shape=B.PROBE_WRITE, dst=dst.data_ptr(), bytes=4096)
    torch.cuda.synchronize()
    assert torch.equal(dst[:1024], torch.tensor([1.0, 2.0, 3.0, 4.0], device=dev).repeat(256)) and (dst[1024:] == -1).all()
    # read only: nothing written
    dst = fresh()
    lib.copy_probe(stream, shape=B.PROBE_READ, src=src.data_ptr(), dst=dst.data_ptr(), bytes=1 << 20)
    torch.cuda.synchronize()
    assert (dst == -1).all()

    # rows of 32768 elements, every grouping of the requests, both pitches on either side
    for group in (1, 2, 4, 8, 16, 32):
        for in_row, out_row in ((32768, 32768), (32768, 32769), (32769, 32768)):
            dst = fresh()
            lib.copy_probe(stream, shape=B.PROBE_ROWS, src=src.data_ptr(), dst=dst.data_ptr(), rows=8,
                           in_row=in_row, out_row=out_row, group=group, workgroups_per_cu=1)
            torch.cuda.synchronize()
            s2 = src[: 8 * in_row * 2].view(8, in_row, 2)[:, :32768]
            d2 = dst[: 8 * out_row * 2].view(8, out_row, 2)
            assert torch.equal(d2[:, :32768], s2), (group, in_row, out_row)
            if out_row > 32768:
                assert (d2[:, 32768:] == -1).all()

    # tiles of 64 x 64 elements of 8 bytes in two slabs of 64 rows of 4096, with each of the numberings
    for extra in ({}, {"xcd_ranges": 1}, {"resident_grid": 1}, {"nontemporal": 1}):
        dst = fresh()
        lib.copy_probe(stream, shape=B.PROBE_TILES, src=src.data_ptr(), dst=dst.data_ptr(), tile_width=64,
                       elem_bytes=8, in_row=4096, out_row=4096, tiles_per_slab=64, rows=2, in_slab=64 * 4096,
                       out_slab=64 * 4096, **extra)
        torch.cuda.synchronize()
        m = 2 * 64 * 4096 * 2
        assert torch.equal(dst[:m], src[:m]) and (dst[m:] == -1).all(), extra
    # rows of a tile 16 rows apart, slabs in two levels (4 slabs a row apart, 2 groups of 64 rows), 16-byte elements
    dst = fresh()
    lib.copy_probe(stream, shape=B.PROBE_TILES, src=src.data_ptr(), dst=dst.data_ptr(), tile_width=8, elem_bytes=16,
                   in_row=4 * 16, out_row=4 * 16, tiles_per_slab=2, rows=8, in_slab=16, out_slab=16,
                   slabs_inner=4, in_slab_outer=4 * 16 * 512, out_slab_outer=4 * 16 * 512)
    torch.cuda.synchronize()
    m = 2 * 4 * 16 * 512 * 4  # two groups of 512 x 4 rows of 16 elements of four floats
    assert torch.equal(dst[:m], src[:m]) and (dst[m:] == -1).all()

    # refused: a byte count that is no multiple of 16, no destination, rows shorter than 32768
    for bad in (dict(shape=B.PROBE_STREAM, src=src.data_ptr(), dst=dst.data_ptr(), bytes=100),
                dict(shape=B.PROBE_STREAM, src=src.data_ptr(), dst=0, bytes=1024),
                dict(shape=B.PROBE_ROWS, src=src.data_ptr(), dst=dst.data_ptr(), rows=2, in_row=1000, out_row=32768),
                dict(shape=B.PROBE_TILES, src=src.data_ptr(), dst=dst.data_ptr(), tile_width=48, elem_bytes=8,
                     in_row=64, out_row=64, tiles_per_slab=1, rows=1),
                dict(shape=99, src=src.data_ptr(), dst=dst.data_ptr(), bytes=1024)):
        with pytest.raises(B.RocfftError):
            lib.copy_probe(stream, **bad)
