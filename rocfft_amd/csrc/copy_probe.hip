// copy_probe.hip -- plain copies in the access shapes of this library's passes.
//
// An FFT pass reads every element once and writes it once, so the rate of a plain copy in the
// same access shape (same workgroup size, same bytes per lane, same strides between the rows of
// a tile) is what the memory system offers that pass; the benchmark prices each kernel against
// the HBM peak and, with these probes, against the copy of its shape.  Nothing here is used by
// a transform.
#include "gpu_rt.h"
#include "rocfft_amd.h"
#include <hip/hip_runtime.h>
#include <algorithm>
#include <stdint.h>

namespace
{

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));

template <typename V>
__device__ __forceinline__ V probe_load(const V* p, bool nt)
{
    return nt ? __builtin_nontemporal_load(p) : *p;
}
template <typename V>
__device__ __forceinline__ void probe_store(V* p, V v, bool nt)
{
    if(nt)
        __builtin_nontemporal_store(v, p);
    else
        *p = v;
}

// 16 bytes per lane, grid-stride
__global__ __launch_bounds__(256) void probe_stream(const v4f* __restrict__ in, v4f* __restrict__ out, size_t n,
                                                    int nt)
{
    for(size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
        probe_store(out + i, probe_load(in + i, nt != 0), nt != 0);
}
__global__ __launch_bounds__(256) void probe_read(const v4f* __restrict__ in, float* out, size_t n)
{
    float acc = 0;
    for(size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    {
        v4f v = in[i];
        acc += v.x + v.y + v.z + v.w;
    }
    if(acc == 12345.678f)
        out[0] = acc;
}
__global__ __launch_bounds__(256) void probe_write(v4f* __restrict__ out, size_t n)
{
    for(size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    {
        v4f c = {1, 2, 3, 4};
        out[i] = c;
    }
}

// The one-workgroup 32768-point kernel's shape: 1024 threads move one row of 32768 elements of
// 8 bytes, 32 per thread, GROUP loads then GROUP stores at a time; rows in_pitch / out_pitch
// elements apart; a resident grid strides through the rows.
template <int GROUP>
__global__ __launch_bounds__(1024) void probe_rows(const v2f* in, v2f* out, size_t in_pitch, size_t out_pitch,
                                                   uint32_t rows, int nt)
{
    for(uint32_t b = blockIdx.x; b < rows; b += gridDim.x)
    {
        const v2f* a = in + (size_t)b * in_pitch;
        v2f*       o = out + (size_t)b * out_pitch;
        v2f        r[GROUP];
        for(int c = 0; c < 32; c += GROUP)
        {
#pragma unroll
            for(int k = 0; k < GROUP; ++k)
                r[k] = probe_load(a + 1024 * (c + k) + threadIdx.x, nt != 0);
#pragma unroll
            for(int k = 0; k < GROUP; ++k)
                probe_store(o + 1024 * (c + k) + threadIdx.x, r[k], nt != 0);
        }
    }
}

// A tile pass's shape: a workgroup of 256 threads moves a tile of W x (4096 / W) elements
// (W neighbouring elements are contiguous, the rows of the tile are in_row / out_row elements
// apart), 16 elements per thread, all loads and then all stores; tiles are numbered along the
// contiguous axis first (tiles_per_slab of them), then by slab (in_slab / out_slab elements apart;
// with slabs_inner set, in two levels: slabs_inner slabs that far apart, groups of them
// in_outer / out_outer apart).
template <typename V>
__global__ __launch_bounds__(256) void probe_tiles(const V* in, V* out, uint32_t W, size_t in_row, size_t out_row,
                                                   uint32_t tiles_per_slab, size_t in_slab, size_t out_slab,
                                                   uint32_t total, int nt, int xcd_ranges, uint32_t slabs_inner,
                                                   size_t in_outer, size_t out_outer)
{
    const uint32_t w = threadIdx.x % W, q = threadIdx.x / W, step = 256 / W;
    for(uint32_t b0 = blockIdx.x; b0 < total; b0 += gridDim.x)
    {
        uint32_t b = b0;
        if(xcd_ranges)
        {
            // workgroups are dealt round-robin to the 8 XCDs: give each XCD one contiguous range of tiles
            const uint32_t xcd = b0 & 7u, idx = b0 >> 3, qd = total >> 3, rm = total & 7u;
            b = xcd * qd + (xcd < rm ? xcd : rm) + idx;
        }
        const uint32_t tile = b % tiles_per_slab, slab = b / tiles_per_slab;
        const uint32_t s_hi = slabs_inner ? slab / slabs_inner : 0, s_lo = slab - s_hi * slabs_inner;
        const V*       a    = in + (size_t)s_lo * in_slab + (size_t)s_hi * in_outer + (size_t)tile * W + w;
        V*             o    = out + (size_t)s_lo * out_slab + (size_t)s_hi * out_outer + (size_t)tile * W + w;
        V              r[16];
#pragma unroll
        for(int k = 0; k < 16; ++k)
            r[k] = probe_load(a + (size_t)(q + step * k) * in_row, nt != 0);
#pragma unroll
        for(int k = 0; k < 16; ++k)
            probe_store(o + (size_t)(q + step * k) * out_row, r[k], nt != 0);
    }
}

int compute_units()
{
    int dev = 0, n = 0;
    if(hipGetDevice(&dev) != hipSuccess
       || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return 0;
    return n;
}

} // namespace

extern "C" int fftrt_copy_probe(const struct rocfft_amd_probe* q, void* stream)
{
    hipStream_t s   = (hipStream_t)stream;
    const int   cus = compute_units();
    if(cus <= 0 || !q || !q->dst)
        return (int)hipErrorInvalidValue;
    const uint32_t per_cu = q->workgroups_per_cu ? q->workgroups_per_cu : 4;
    switch(q->shape)
    {
    case ROCFFT_AMD_PROBE_STREAM:
    {
        if(!q->src || q->bytes % 16)
            return (int)hipErrorInvalidValue;
        const size_t   n    = q->bytes / 16;
        const uint32_t grid = (uint32_t)std::min<size_t>((n + 255) / 256, (size_t)per_cu * cus);
        hipLaunchKernelGGL(probe_stream, dim3(grid), dim3(256), 0, s, static_cast<const v4f*>(q->src),
                           static_cast<v4f*>(q->dst), n, q->nontemporal);
        break;
    }
    case ROCFFT_AMD_PROBE_READ:
    {
        if(!q->src || q->bytes % 16)
            return (int)hipErrorInvalidValue;
        const size_t   n    = q->bytes / 16;
        const uint32_t grid = (uint32_t)std::min<size_t>((n + 255) / 256, (size_t)per_cu * cus);
        hipLaunchKernelGGL(probe_read, dim3(grid), dim3(256), 0, s, static_cast<const v4f*>(q->src),
                           static_cast<float*>(q->dst), n);
        break;
    }
    case ROCFFT_AMD_PROBE_WRITE:
    {
        if(q->bytes % 16)
            return (int)hipErrorInvalidValue;
        const size_t   n    = q->bytes / 16;
        const uint32_t grid = (uint32_t)std::min<size_t>((n + 255) / 256, (size_t)per_cu * cus);
        hipLaunchKernelGGL(probe_write, dim3(grid), dim3(256), 0, s, static_cast<v4f*>(q->dst), n);
        break;
    }
    case ROCFFT_AMD_PROBE_ROWS:
    {
        // rows of 32768 elements of 8 bytes
        if(!q->src || q->rows == 0 || q->in_row < 32768 || q->out_row < 32768)
            return (int)hipErrorInvalidValue;
        const uint32_t grid = std::min<uint32_t>(q->rows, per_cu * (uint32_t)cus);
        const v2f* src = static_cast<const v2f*>(q->src);
        v2f*       dst = static_cast<v2f*>(q->dst);
#define PROBE_ROWS_GROUP(G)                                                                                      \
    hipLaunchKernelGGL(probe_rows<G>, dim3(grid), dim3(1024), 0, s, src, dst, q->in_row, q->out_row, q->rows, \
                       q->nontemporal)
        switch(q->group)
        {
        case 1: PROBE_ROWS_GROUP(1); break;
        case 2: PROBE_ROWS_GROUP(2); break;
        case 4: PROBE_ROWS_GROUP(4); break;
        case 8: PROBE_ROWS_GROUP(8); break;
        case 16: PROBE_ROWS_GROUP(16); break;
        default: PROBE_ROWS_GROUP(32); break;
        }
#undef PROBE_ROWS_GROUP
        break;
    }
    case ROCFFT_AMD_PROBE_TILES:
    {
        const uint32_t W = q->tile_width;
        if(!q->src || W == 0 || W > 256 || (W & (W - 1)) || q->rows == 0 || q->tiles_per_slab == 0)
            return (int)hipErrorInvalidValue;
        const uint64_t total = (uint64_t)q->tiles_per_slab * q->rows; // rows = slabs here
        if(total >= (1ull << 31))
            return (int)hipErrorInvalidValue;
        const uint32_t grid = (uint32_t)std::min<uint64_t>(total, q->resident_grid ? (uint64_t)per_cu * cus : total);
        const int      xcd  = (q->xcd_ranges && grid == total) ? 1 : 0;
        if(q->elem_bytes == 8)
            hipLaunchKernelGGL(probe_tiles<v2f>, dim3(grid), dim3(256), 0, s, static_cast<const v2f*>(q->src),
                               static_cast<v2f*>(q->dst), W, q->in_row, q->out_row, q->tiles_per_slab, q->in_slab,
                               q->out_slab, (uint32_t)total, q->nontemporal, xcd, q->slabs_inner, q->in_slab_outer,
                               q->out_slab_outer);
        else if(q->elem_bytes == 16)
            hipLaunchKernelGGL(probe_tiles<v4f>, dim3(grid), dim3(256), 0, s, static_cast<const v4f*>(q->src),
                               static_cast<v4f*>(q->dst), W, q->in_row, q->out_row, q->tiles_per_slab, q->in_slab,
                               q->out_slab, (uint32_t)total, q->nontemporal, xcd, q->slabs_inner, q->in_slab_outer,
                               q->out_slab_outer);
        else
            return (int)hipErrorInvalidValue;
        break;
    }
    default:
        return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}
