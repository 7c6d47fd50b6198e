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
 * with rocfft_plan_get_work_buffer_size); load/store callbacks and half
 * precision, which stage through per-call buffers, return
 * rocfft_status_failure.  All calls on one GPU share the one array: calls that
 * overlap in time on the same GPU (different streams or threads) race.
 * Nothing in the array has to be cleared between calls (every pass writes the
 * part of the work area it later reads).
 */
#define ROCFFT_AMD_STATIC_WORK_BYTES ((size_t)64 << 20)
ROCFFT_EXPORT rocfft_status rocfft_amd_execute_static(const rocfft_plan     plan,
                                                      void*                 in_buffer[],
                                                      void*                 out_buffer[],
                                                      rocfft_execution_info info);

#ifdef __cplusplus
}
#endif
#endif
