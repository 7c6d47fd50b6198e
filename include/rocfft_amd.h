/*
 * rocfft_amd.h -- entry points this library adds to the rocfft.h interface.
 * They have no counterpart in the reference.
 */
#ifndef ROCFFT_AMD_H
#define ROCFFT_AMD_H

#include "rocfft/rocfft.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Plans a transform exactly as rocfft_plan_create would, without touching a
 * device, and writes the pass list as text (the same text rocfft_plan_get_print
 * prints; reference rocfft.h:443 / library/src/plan.cpp:4476-4514 is the
 * nearest counterpart).  text may be NULL.  work_buffer_bytes, when not NULL,
 * receives what rocfft_plan_get_work_buffer_size would report.  Returns the
 * status rocfft_plan_create would return for the same arguments, apart from
 * device errors.
 */
ROCFFT_EXPORT rocfft_status rocfft_amd_plan_describe(rocfft_result_placement       placement,
                                                     rocfft_transform_type         transform_type,
                                                     rocfft_precision              precision,
                                                     size_t                        dimensions,
                                                     const size_t*                 lengths,
                                                     size_t                        number_of_transforms,
                                                     const rocfft_plan_description description,
                                                     char*                         text,
                                                     size_t                        text_len,
                                                     size_t*                       work_buffer_bytes);

/*
 * Per-pass profiling, the counterpart of the reference's profile log layer
 * (library/src/powX.cpp:817-883 brackets every kernel with hipEvents when
 * ROCFFT_LAYER has the profile bit).  A plan is a short list of passes, one
 * kernel launch each.
 */
ROCFFT_EXPORT rocfft_status rocfft_amd_plan_get_pass_count(const rocfft_plan plan, size_t* count);

/* Name of pass `index` and the data bytes it reads plus writes (tables excluded). */
ROCFFT_EXPORT rocfft_status rocfft_amd_plan_get_pass_info(const rocfft_plan plan,
                                                          size_t            index,
                                                          char*             name,
                                                          size_t            name_len,
                                                          double*           bytes_read_written);

/*
 * rocfft_execute with every pass bracketed by events on the execution stream;
 * waits for the stream and writes one duration in milliseconds per pass.
 * capacity must be at least the pass count.  Not usable during graph capture.
 */
ROCFFT_EXPORT rocfft_status rocfft_amd_execute_profile(const rocfft_plan     plan,
                                                       void*                 in_buffer[],
                                                       void*                 out_buffer[],
                                                       rocfft_execution_info info,
                                                       float*                pass_ms,
                                                       size_t                capacity);

/*
 * rocfft_execute for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  The plan's work area is a device-resident
 * array of ROCFFT_AMD_STATIC_WORK_BYTES that the library holds on every GPU it
 * runs on until the process ends; a work buffer set in `info` is ignored, its
 * stream is used.  The call allocates and frees nothing.  Plans that need a
 * larger work area return rocfft_status_invalid_work_buffer (query the need
 * with rocfft_plan_get_work_buffer_size).  Load/store callbacks are accepted
 * when the first and last kernel of the plan call them themselves, and
 * half-precision plans when their kernels read and write the half arrays
 * themselves and need no single-precision copy of either array (one-kernel
 * plans over interleaved arrays); executions that would have to stage an array
 * through a buffer of the plan's return rocfft_status_failure unless an
 * earlier rocfft_execute on the same stream has already allocated it.  All
 * calls on one GPU share the one array: calls that overlap in time on the same
 * GPU (different streams or threads) race.  Nothing in the array has to be
 * cleared between calls (every pass writes the part of the work area it later
 * reads).
 */
#define ROCFFT_AMD_STATIC_WORK_BYTES ((size_t)64 << 20)
ROCFFT_EXPORT rocfft_status rocfft_amd_execute_static(const rocfft_plan     plan,
                                                      void*                 in_buffer[],
                                                      void*                 out_buffer[],
                                                      rocfft_execution_info info);

/*
 * Plain copies in the access shapes of this library's passes, for measurement: an FFT pass
 * reads every element once and writes it once, so a copy with the same workgroup size, bytes
 * per lane and strides is what the memory system offers that pass.  The call enqueues one
 * copy kernel on `stream`; time it with events.  It has no counterpart in the reference.
 */
enum rocfft_amd_probe_shape
{
    ROCFFT_AMD_PROBE_STREAM = 0, /* bytes from src to dst, 16 bytes per lane, resident grid-stride loop */
    ROCFFT_AMD_PROBE_READ   = 1, /* reads `bytes` of src (dst: 4 bytes that are never written) */
    ROCFFT_AMD_PROBE_WRITE  = 2, /* writes `bytes` of dst */
    ROCFFT_AMD_PROBE_ROWS   = 3, /* `rows` rows of 32768 elements of 8 bytes, one workgroup of 1024 threads per
                                    row, `group` (8 or 32) loads then as many stores at a time; rows in_row /
                                    out_row elements apart */
    ROCFFT_AMD_PROBE_TILES  = 4  /* tiles of tile_width x (4096 / tile_width) elements of elem_bytes (8 or 16),
                                    one workgroup of 256 threads per tile, 16 loads then 16 stores per thread;
                                    tile rows in_row / out_row elements apart; tiles_per_slab tiles side by
                                    side, `rows` slabs in_slab / out_slab elements apart */
};
typedef struct rocfft_amd_probe
{
    int         shape;
    const void* src;
    void*       dst;
    size_t      bytes;
    int         nontemporal;       /* loads and stores carry the nontemporal hint */
    unsigned    workgroups_per_cu; /* resident grids: workgroups per compute unit (0 = 4) */
    unsigned    group;
    unsigned    rows;
    size_t      in_row, out_row;
    unsigned    tile_width, elem_bytes, tiles_per_slab;
    size_t      in_slab, out_slab;
    int         resident_grid; /* tiles: 1 = a resident grid strides through the tiles, 0 = one workgroup per tile */
    int         xcd_ranges;    /* tiles, one workgroup per tile: 1 = workgroups renumbered so that each of the 8 XCDs
                                  works through one contiguous range of tiles, as the column passes do */
    unsigned    slabs_inner;   /* tiles: not 0 = slab s starts at (s % slabs_inner) * in_slab + (s / slabs_inner) *
                                  in_slab_outer (out likewise) instead of s * in_slab */
    size_t      in_slab_outer, out_slab_outer;
} rocfft_amd_probe;
ROCFFT_EXPORT rocfft_status rocfft_amd_copy_probe(const rocfft_amd_probe* probe, void* stream);

#ifdef __cplusplus
}
#endif
#endif
