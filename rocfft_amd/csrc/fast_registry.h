// fast_registry.h -- table entry of a compile-time-schedule tile kernel.  Each slice of
// fast_kernels.hip exports its entries; the lookup (fast_kernels.hip, slice 0) merges them.
#ifndef ROCFFT_AMD_FAST_REGISTRY_H
#define ROCFFT_AMD_FAST_REGISTRY_H

#include "kparams.h"
#include <stddef.h>
#include <stdint.h>

typedef int (*fast_launch_fn)(const struct fftk_params*, uint32_t grid, size_t lds_bytes, void* stream);

struct FastEntry
{
    int      precision; // 0 single, 1 double
    uint32_t n;
    uint32_t radix[4]; // unused passes are 1
    uint32_t tpt; // threads per transform
    // lean: vector accesses, interleaved complex on both sides; vec: vector accesses, every
    // fused operation; scalar: scalar accesses.  A missing variant is null and the generic
    // kernel runs instead.
    fast_launch_fn lean, vec, scalar;
    // the lean kernel compiled for plain passes only, and for the other passes over interleaved
    // arrays without a chirp (twiddle on the store side, real pre/post-processing, tile copies,
    // half-precision arrays on the user's side)
    fast_launch_fn plain, more;
    // the lean kernel compiled for odd-length real transforms (real samples on one side, the half
    // spectrum on the other; odd lengths only)
    fast_launch_fn odd_real;
    // the lean kernel compiled for the first (chirp and padding on the load side, large twiddle on
    // the store side), the last (chirp and scale on the store side) and the middle pass (forward
    // transform, spectrum product, inverse transform, large twiddle) of a chirp-z transform in
    // three kernels; null where none is built
    fast_launch_fn chirp_in, chirp_out, chirp_mid;
};

#endif
