// gpu_rt.h -- the thin C-ABI layer between the host library (planner, API,
// table builders: plain C++) and the GPU (HIP runtime calls and kernel
// launches).  Nothing above this layer includes a HIP header.
//
// Two implementations exist: kernels.hip and the other .hip files (the product, HIP on
// gfx950: a shared library of its own, librocfft_amd_rt.so, which the host library links
// against -- its functions are the only symbols it exports) and
// tests/emu/gpu_rt_emu.cpp (host loops over the same kernel bodies, used only
// by the CPU test-suite to exercise the planner without a GPU).
#ifndef ROCFFT_AMD_GPU_RT_H
#define ROCFFT_AMD_GPU_RT_H

#include "kparams.h"
#include <stddef.h>

#define FFTRT_API __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

// 0 on success, non-zero (the HIP error code) otherwise
FFTRT_API int fftrt_device_count(int* count);
FFTRT_API int fftrt_device_info(int* device, int* compute_units, int* lds_bytes, char* arch, size_t arch_len);
FFTRT_API int fftrt_malloc(void** ptr, size_t bytes);
FFTRT_API int fftrt_free(void* ptr);
FFTRT_API int fftrt_upload(void* dst, const void* src, size_t bytes);
FFTRT_API int fftrt_download(void* dst, const void* src, size_t bytes);
FFTRT_API int fftrt_stream_sync(void* stream);
FFTRT_API int fftrt_device_sync(void);
// 1 when `stream` is being captured into a graph
FFTRT_API int fftrt_stream_capturing(void* stream);

// Pass schedule of the compile-time-schedule ("fast") kernel for length n: writes its
// radices (at most 4) and their count and returns its threads per transform, or returns 0
// when there is no such kernel (the generic kernel runs the planner's own factorisation
// then).  The threads per transform follow the generic kernel's rule, so a pass planned
// for a fast kernel can run on the generic one when an access mode has no fast variant.
FFTRT_API uint32_t fftrt_fast_schedule(int precision, uint32_t n, uint32_t* radix, uint32_t* nf);
// 1 when a compiled single-precision kernel of length n can read or write arrays of IEEE half
// pairs (the user's arrays of a half-precision plan)
FFTRT_API int fftrt_fast_takes_half(uint32_t n);
// returned by the fast launcher when the requested access mode has no compiled variant
#define FFTRT_NO_FAST_VARIANT (-2)

// precision: 0 = float, 1 = double.  vec: 1 when both sides are interleaved
// complex and can move (re, im) pairs with one access.
FFTRT_API int fftrt_launch_tile(const struct fftk_params* p, int precision, int vec, uint32_t grid,
                      size_t lds_bytes, void* stream);
FFTRT_API int fftrt_launch_real_post(const struct fftk_real_params* p, int precision, void* stream);
FFTRT_API int fftrt_launch_real_pre(const struct fftk_real_params* p, int precision, void* stream);
FFTRT_API int fftrt_launch_copy(const struct fftk_copy_params* p, int precision, void* stream);
// complex_elems: 1 = the array holds (re, im) pairs, 0 = real scalars
FFTRT_API int fftrt_launch_callback_copy(const struct fftk_cb_params* p, int precision, int complex_elems, void* stream);
// the same copy between a half-precision user array and a single-precision scratch array
FFTRT_API int fftrt_launch_half_copy(const struct fftk_cb_params* p, int complex_elems, void* stream);

// One-workgroup 2D kernel for small nA x nB complex transforms (nA the unit-stride dimension):
// fftrt_fast2d_info returns 0 when there is none for these sizes, else 1 and the two pass
// schedules, their threads per transform and the LDS pitch between rows.  The launch takes
// p->n = nA, p->n2 = nB, p->W transforms per workgroup, p->tw / p->tw2 the twiddle tables.
FFTRT_API int fftrt_fast2d_info(uint32_t nA, uint32_t nB, uint32_t* radixA, uint32_t* nfA, uint32_t* radixB,
                      uint32_t* nfB, uint32_t* tptA, uint32_t* tptB, uint32_t* pitchA);
FFTRT_API int fftrt_launch_fast2d(const struct fftk_params* p, int precision, uint32_t grid, size_t lds_bytes, void* stream);
// The same for real transforms of 2L x nB points (p->n = L, the half length; p->half_tw its
// post-/pre-processing twiddles): forward reads real rows and writes L+1 bins per row, inverse the
// other way round.  `pitch` is the LDS pitch between the rows of L+1 bins.
FFTRT_API int fftrt_fast2d_real_info(uint32_t L, uint32_t nB, uint32_t* radixA, uint32_t* nfA, uint32_t* radixB,
                           uint32_t* nfB, uint32_t* tptA, uint32_t* tptB, uint32_t* pitch);
FFTRT_API int fftrt_launch_fast2d_real(const struct fftk_params* p, int precision, int inverse, uint32_t grid,
                             size_t lds_bytes, void* stream);

// 1 when the one-workgroup 32768-point kernel is available in this runtime
FFTRT_API int fftrt_has_big32k(void);
FFTRT_API int fftrt_launch_big32k(const struct fftk_big_params* p, void* stream);

// Device-resident work area that exists for the life of the process (one copy per
// device): its address on the current device and its size.  Used by the execute
// variant that may not allocate.  Calls that use it at the same time on one device race.
#define FFTRT_STATIC_SCRATCH_BYTES (64u << 20)
FFTRT_API int fftrt_static_scratch(void** ptr, size_t* bytes);

// plain copies in the access shapes of the passes (rocfft_amd.h: rocfft_amd_copy_probe)
struct rocfft_amd_probe;
FFTRT_API int fftrt_copy_probe(const struct rocfft_amd_probe* q, void* stream);

// event timing, used by the optional per-pass profile log
FFTRT_API int fftrt_event_create(void** ev);
FFTRT_API int fftrt_event_destroy(void* ev);
FFTRT_API int fftrt_event_record(void* ev, void* stream);
FFTRT_API int fftrt_event_elapsed_ms(void* start, void* stop, float* ms);

#ifdef __cplusplus
}
#endif
#endif
