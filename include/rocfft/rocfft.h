/*
 * rocfft.h -- public C interface of the MI355X-native FFT library.
 *
 * Every identifier, enumerator value and function signature below is binary
 * compatible with the reference interface it replaces
 * (reference: library/include/rocfft/rocfft.h; the line each entry point
 * replaces is cited beside it), so a program built against the reference
 * header can be pointed at this library without recompiling.
 *
 * Conventions (reference rocfft.h:161-164, 201-209; plan.cpp:87-197):
 *   - lengths[0] is the fastest-varying dimension;
 *   - transforms are unnormalised in both directions;
 *   - strides, distances and offsets count elements of the array's own type;
 *   - in_buffer/out_buffer are arrays of device pointers, one entry for
 *     interleaved and real arrays, two (real part, imaginary part) for planar;
 *   - rocfft_execute only enqueues work on the stream of the execution info
 *     (the null stream by default) and returns without waiting for it.
 */
#ifndef ROCFFT_H
#define ROCFFT_H

#ifndef ROCFFT_EXPORT
#define ROCFFT_EXPORT __attribute__((visibility("default")))
#endif

#ifdef __cplusplus
#include <cstddef>
extern "C" {
#else
#include <stddef.h>
#endif

/* Opaque handles (reference rocfft.h:45-69). */
typedef struct rocfft_plan_t*             rocfft_plan;
typedef struct rocfft_plan_description_t* rocfft_plan_description;
typedef struct rocfft_execution_info_t*   rocfft_execution_info;
typedef struct rocfft_field_t*            rocfft_field;
typedef struct rocfft_brick_t*            rocfft_brick;

/* Status codes, values 0..8 (reference rocfft.h:77-88). */
typedef enum rocfft_status_e
{
    rocfft_status_success             = 0,
    rocfft_status_failure             = 1,
    rocfft_status_invalid_arg_value   = 2,
    rocfft_status_invalid_dimensions  = 3,
    rocfft_status_invalid_array_type  = 4,
    rocfft_status_invalid_strides     = 5,
    rocfft_status_invalid_distance    = 6,
    rocfft_status_invalid_offset      = 7,
    rocfft_status_invalid_work_buffer = 8
} rocfft_status;

/* Transform kinds, values 0..3 (reference rocfft.h:91-97). */
typedef enum rocfft_transform_type_e
{
    rocfft_transform_type_complex_forward = 0,
    rocfft_transform_type_complex_inverse = 1,
    rocfft_transform_type_real_forward    = 2,
    rocfft_transform_type_real_inverse    = 3
} rocfft_transform_type;

/* Precision (reference rocfft.h:100-105). Half precision keeps the layouts of
   the plan description; its arrays hold IEEE half values, the arithmetic runs in
   single precision on copies the plan owns and the result is rounded back. */
typedef enum rocfft_precision_e
{
    rocfft_precision_single = 0,
    rocfft_precision_double = 1,
    rocfft_precision_half   = 2
} rocfft_precision;

/* Placement (reference rocfft.h:113-117). An out-of-place real inverse
   transform may overwrite its input; no other out-of-place transform does. */
typedef enum rocfft_result_placement_e
{
    rocfft_placement_inplace    = 0,
    rocfft_placement_notinplace = 1
} rocfft_result_placement;

/* Array formats (reference rocfft.h:120-128). */
typedef enum rocfft_array_type_e
{
    rocfft_array_type_complex_interleaved   = 0,
    rocfft_array_type_complex_planar        = 1,
    rocfft_array_type_real                  = 2,
    rocfft_array_type_hermitian_interleaved = 3,
    rocfft_array_type_hermitian_planar      = 4,
    rocfft_array_type_unset                 = 5
} rocfft_array_type;

/* Communicator kinds for distributed plans (reference rocfft.h:131-135). */
typedef enum rocfft_comm_type_e
{
    rocfft_comm_none = 0,
    rocfft_comm_mpi  = 1
} rocfft_comm_type;

/* Library set-up / tear-down; may be called repeatedly (reference rocfft.h:149,153). */
ROCFFT_EXPORT rocfft_status rocfft_setup(void);
ROCFFT_EXPORT rocfft_status rocfft_cleanup(void);

/* Build a plan for `number_of_transforms` transforms of `dimensions` (1..3)
   dimensions (reference rocfft.h:188-195).  `description` may be NULL. */
ROCFFT_EXPORT rocfft_status rocfft_plan_create(rocfft_plan*                  plan,
                                               rocfft_result_placement       placement,
                                               rocfft_transform_type         transform_type,
                                               rocfft_precision              precision,
                                               size_t                        dimensions,
                                               const size_t*                 lengths,
                                               size_t                        number_of_transforms,
                                               const rocfft_plan_description description);

/* Enqueue the transform (reference rocfft.h:231-234).  out_buffer may be NULL
   for in-place plans; info may be NULL. */
ROCFFT_EXPORT rocfft_status rocfft_execute(const rocfft_plan     plan,
                                           void*                 in_buffer[],
                                           void*                 out_buffer[],
                                           rocfft_execution_info info);

/* reference rocfft.h:240 */
ROCFFT_EXPORT rocfft_status rocfft_plan_destroy(rocfft_plan plan);

/* Multiply every output element by a finite factor (reference rocfft.h:250). */
ROCFFT_EXPORT rocfft_status rocfft_plan_description_set_scale_factor(
    rocfft_plan_description description, const double scale_factor);

/* Array formats, offsets, strides and batch distances (reference
   rocfft.h:296-307).  NULL pointers / zero distances keep the defaults. */
ROCFFT_EXPORT rocfft_status
    rocfft_plan_description_set_data_layout(rocfft_plan_description description,
                                            const rocfft_array_type in_array_type,
                                            const rocfft_array_type out_array_type,
                                            const size_t*           in_offsets,
                                            const size_t*           out_offsets,
                                            const size_t            in_strides_size,
                                            const size_t*           in_strides,
                                            const size_t            in_distance,
                                            const size_t            out_strides_size,
                                            const size_t*           out_strides,
                                            const size_t            out_distance);

/* Distributed-transform entry points (reference rocfft.h:313-322, 344,
   378-389, 405, 416-429).  This library drives one GPU: handles can be
   created and destroyed, but attaching a field or an MPI communicator to a
   description makes plan creation return rocfft_status_failure. */
ROCFFT_EXPORT rocfft_status rocfft_field_create(rocfft_field* field);
ROCFFT_EXPORT rocfft_status rocfft_field_destroy(rocfft_field field);

/* reference rocfft.h:329 */
ROCFFT_EXPORT rocfft_status rocfft_get_version_string(char* buf, size_t len);

ROCFFT_EXPORT rocfft_status rocfft_plan_description_set_comm(rocfft_plan_description description,
                                                             rocfft_comm_type        comm_type,
                                                             void*                   comm_handle);
ROCFFT_EXPORT rocfft_status rocfft_brick_create(rocfft_brick* brick,
                                                const size_t* field_lower,
                                                const size_t* field_upper,
                                                const size_t* brick_stride,
                                                size_t        dim,
                                                int           deviceID);
ROCFFT_EXPORT rocfft_status rocfft_brick_destroy(rocfft_brick brick);
ROCFFT_EXPORT rocfft_status rocfft_field_add_brick(rocfft_field field, rocfft_brick brick);
ROCFFT_EXPORT rocfft_status rocfft_plan_description_add_infield(rocfft_plan_description description,
                                                                rocfft_field            field);
ROCFFT_EXPORT rocfft_status
    rocfft_plan_description_add_outfield(rocfft_plan_description description, rocfft_field field);

/* Bytes of device scratch the plan needs at execute (reference rocfft.h:436). */
ROCFFT_EXPORT rocfft_status rocfft_plan_get_work_buffer_size(const rocfft_plan plan,
                                                             size_t*           size_in_bytes);

/* Print the pass list of the plan to stdout (reference rocfft.h:443). */
ROCFFT_EXPORT rocfft_status rocfft_plan_get_print(const rocfft_plan plan);

/* reference rocfft.h:450-457 */
ROCFFT_EXPORT rocfft_status rocfft_plan_description_create(rocfft_plan_description* description);
ROCFFT_EXPORT rocfft_status rocfft_plan_description_destroy(rocfft_plan_description description);

/* reference rocfft.h:465-473 */
ROCFFT_EXPORT rocfft_status rocfft_execution_info_create(rocfft_execution_info* info);
ROCFFT_EXPORT rocfft_status rocfft_execution_info_destroy(rocfft_execution_info info);

/* Caller-owned scratch for rocfft_execute (reference rocfft.h:501).  Without
   one, execute allocates and frees scratch itself when the plan needs any. */
ROCFFT_EXPORT rocfft_status rocfft_execution_info_set_work_buffer(rocfft_execution_info info,
                                                                  void*                 work_buffer,
                                                                  const size_t size_in_bytes);

/* hipStream_t to enqueue on (reference rocfft.h:530). */
ROCFFT_EXPORT rocfft_status rocfft_execution_info_set_stream(rocfft_execution_info info,
                                                             void*                 stream);

/* User load/store device callbacks (reference rocfft.h:533-612):
     T    load_cb (T* data, size_t offset, void* cbdata, void* sharedMem);
     void store_cb(T* data, size_t offset, T element, void* cbdata, void* sharedMem);
   T is the element type of the input (output) array, offset counts such elements from the
   buffer pointer given to rocfft_execute.  cb_functions[0] / cb_data[0] are used (one
   device); a null function clears the callback; shared_mem_bytes must be 0
   (rocfft_status_invalid_arg_value otherwise).  An execute with callbacks fails for planar
   arrays and during stream capture. */
ROCFFT_EXPORT rocfft_status rocfft_execution_info_set_load_callback(rocfft_execution_info info,
                                                                    void** cb_functions,
                                                                    void** cb_data,
                                                                    size_t shared_mem_bytes);
ROCFFT_EXPORT rocfft_status rocfft_execution_info_set_store_callback(rocfft_execution_info info,
                                                                     void** cb_functions,
                                                                     void** cb_data,
                                                                     size_t shared_mem_bytes);

/* Compiled-kernel cache (reference rocfft.h:632-646).  Kernels are compiled
   ahead of time here, so the cache is always empty: serialize yields a
   zero-length buffer and deserialize accepts anything. */
ROCFFT_EXPORT rocfft_status rocfft_cache_serialize(void** buffer, size_t* buffer_len_bytes);
ROCFFT_EXPORT rocfft_status rocfft_cache_buffer_free(void* buffer);
ROCFFT_EXPORT rocfft_status rocfft_cache_deserialize(const void* buffer, size_t buffer_len_bytes);

#ifdef __cplusplus
}
#endif

#endif /* ROCFFT_H */
