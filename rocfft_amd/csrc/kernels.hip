// kernels.hip -- gfx950 kernels and the HIP side of the C-ABI runtime layer.
#include "gpu_rt.h"
#include "lds_limit.h"
#include "tile_core.h"
#include <hip/hip_runtime.h>
#include <mutex>
#include <string.h>

namespace
{

template <typename T>
__device__ __forceinline__ void run_passes(const fftk_params&         p,
                                           typename cplx_of<T>::type* lds,
                                           uint32_t                   w,
                                           uint32_t                   tt,
                                           bool                       active)
{
    typedef typename cplx_of<T>::type C;
    for(uint32_t pass = 0; pass < p.nf; ++pass)
    {
        C r[FFTK_REG_ELEMS];
        switch(p.radix[pass])
        {
#define FFTK_CASE(R)                                         \
    case R:                                                  \
        pass_read<T, R>(p, lds, w, tt, active, r);           \
        __syncthreads();                                     \
        pass_write<T, R>(p, (int)pass, lds, w, tt, active, r); \
        break;
            FFTK_CASE(2)
            FFTK_CASE(3)
            FFTK_CASE(4)
            FFTK_CASE(5)
            FFTK_CASE(6)
            FFTK_CASE(7)
            FFTK_CASE(8)
            FFTK_CASE(9)
            FFTK_CASE(10)
            FFTK_CASE(11)
            FFTK_CASE(12)
            FFTK_CASE(13)
            FFTK_CASE(14)
            FFTK_CASE(15)
            FFTK_CASE(16)
            FFTK_CASE(17)
#undef FFTK_CASE
        default:
            __syncthreads();
            break;
        }
        __syncthreads();
    }
}

// The row copy and the real pre/post-processing kernels exist twice: CB = true calls the caller's
// load and store callbacks where the parameters name them (indirect calls: the kernel then needs a
// stack and the registers any callee may use), CB = false works on a copy of its parameters
// without callbacks, which lets the compiler drop those calls: 16-26 registers, no stack, eight
// waves a SIMD.  The tile kernel has one form: it takes 256 registers with or without the calls
// (its parameter block is indexed at run time, so a copy of it would live in scratch memory).
template <bool CB, typename P>
__device__ __forceinline__ P callbacks_as_built(const P& given)
{
    P p = given;
    if constexpr(!CB)
    {
        p.cb.load_fn  = nullptr;
        p.cb.store_fn = nullptr;
    }
    return p;
}

template <typename T, bool VEC, int BLK>
__global__ __launch_bounds__(BLK) void tile_fft_kernel(const fftk_params p)
{
    typedef typename cplx_of<T>::type C;
    extern __shared__ double2         smem_raw[];
    C*                                lds = reinterpret_cast<C*>(smem_raw);
    const uint32_t                    tid = threadIdx.x;
    TileCtx<T>                        c;
    tile_decode<T>(p, blockIdx.x, c);
    tile_load<T, VEC>(p, c, lds, tid);
    __syncthreads();
    uint32_t w, tt;
    bool     active;
    thread_role(p, tid, w, tt, active);
    run_passes<T>(p, lds, w, tt, active);
    if(p.flags & FFTK_F_CONV)
    {
        tile_conv<T>(p, c, lds, tid);
        __syncthreads();
        run_passes<T>(p, lds, w, tt, active);
    }
    tile_store<T, VEC>(p, c, lds, tid);
}

template <typename T, bool CB>
__global__ __launch_bounds__(256) void real_post_kernel(const fftk_real_params given)
{
    const fftk_real_params p = callbacks_as_built<CB>(given);
    real_post_elem<T>(p, (uint64_t)blockIdx.x * 256 + threadIdx.x);
}

template <typename E>
__global__ __launch_bounds__(256) void callback_copy_kernel(const fftk_cb_params p)
{
    callback_elem<E>(p, (uint64_t)blockIdx.x * 256 + threadIdx.x);
}

template <typename U, typename E>
__global__ __launch_bounds__(256) void half_copy_kernel(const fftk_cb_params p)
{
    half_stage_elem<U, E>(p, (uint64_t)blockIdx.x * 256 + threadIdx.x);
}

template <typename T, bool CB>
__global__ __launch_bounds__(256) void row_copy_kernel(const fftk_copy_params given)
{
    const fftk_copy_params p = callbacks_as_built<CB>(given);
    copy_elem<T>(p, (uint64_t)blockIdx.x * 256 + threadIdx.x);
}

template <typename T, bool CB>
__global__ __launch_bounds__(256) void real_pre_kernel(const fftk_real_params given)
{
    const fftk_real_params p = callbacks_as_built<CB>(given);
    real_pre_elem<T>(p, (uint64_t)blockIdx.x * 256 + threadIdx.x);
}

constexpr size_t MAX_LDS_BYTES = 160 * 1024;

template <typename P>
bool has_callbacks(const P* p)
{
    return p->cb.load_fn != nullptr || p->cb.store_fn != nullptr;
}

template <typename T, bool VEC, int BLK>
int launch_tile_t(const fftk_params* p, uint32_t grid, size_t lds_bytes, hipStream_t stream)
{
    auto kernel = tile_fft_kernel<T, VEC, BLK>;
    if(lds_bytes > 64 * 1024)
    {
        static FftLdsLimit limit;
        if(int rc = limit.allow(kernel, (int)MAX_LDS_BYTES))
            return rc;
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(p->nthreads), lds_bytes, stream, *p);
    return (int)hipGetLastError();
}

template <typename T, bool VEC>
int launch_tile_b(const fftk_params* p, uint32_t grid, size_t lds_bytes, hipStream_t stream)
{
    if(p->nthreads <= 256)
        return launch_tile_t<T, VEC, 256>(p, grid, lds_bytes, stream);
    return launch_tile_t<T, VEC, 512>(p, grid, lds_bytes, stream);
}

} // namespace

extern "C" {

int fftrt_device_count(int* count)
{
    return (int)hipGetDeviceCount(count);
}

int fftrt_device_info(int* device, int* compute_units, int* lds_bytes, char* arch, size_t arch_len)
{
    int dev = 0;
    int rc  = (int)hipGetDevice(&dev);
    if(rc)
        return rc;
    hipDeviceProp_t prop;
    rc = (int)hipGetDeviceProperties(&prop, dev);
    if(rc)
        return rc;
    if(device)
        *device = dev;
    if(compute_units)
        *compute_units = prop.multiProcessorCount;
    if(lds_bytes)
        *lds_bytes = (int)prop.maxSharedMemoryPerMultiProcessor;
    if(arch && arch_len)
    {
        strncpy(arch, prop.gcnArchName, arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    return 0;
}

int fftrt_malloc(void** ptr, size_t bytes)
{
    return (int)hipMalloc(ptr, bytes);
}
int fftrt_free(void* ptr)
{
    return (int)hipFree(ptr);
}
int fftrt_upload(void* dst, const void* src, size_t bytes)
{
    return (int)hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice);
}
int fftrt_download(void* dst, const void* src, size_t bytes)
{
    return (int)hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost);
}
int fftrt_stream_sync(void* stream)
{
    return (int)hipStreamSynchronize((hipStream_t)stream);
}
int fftrt_device_sync(void)
{
    return (int)hipDeviceSynchronize();
}
int fftrt_stream_capturing(void* stream)
{
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if(hipStreamIsCapturing((hipStream_t)stream, &st) != hipSuccess)
        return 0;
    return st == hipStreamCaptureStatusActive ? 1 : 0;
}

int fftrt_launch_fast_tile(const struct fftk_params* p, int precision, int vec, uint32_t grid,
                           size_t lds_bytes, void* stream);

int fftrt_launch_tile(const struct fftk_params* p, int precision, int vec, uint32_t grid,
                      size_t lds_bytes, void* stream)
{
    hipStream_t s = (hipStream_t)stream;
    if(p->fast)
    {
        if(p->nthreads == 0 || (p->nthreads & 63) || lds_bytes > MAX_LDS_BYTES || grid == 0)
            return (int)hipErrorInvalidValue;
        int rc = fftrt_launch_fast_tile(p, precision, vec, grid, lds_bytes, stream);
        if(rc != FFTRT_NO_FAST_VARIANT)
            return rc;
        // no compiled variant for this access mode: the generic kernel runs the same schedule
    }
    if(p->nthreads == 0 || p->nthreads > 512 || (p->nthreads & 63) || lds_bytes > MAX_LDS_BYTES
       || grid == 0)
        return (int)hipErrorInvalidValue;
    if(precision == 0)
        return vec ? launch_tile_b<float, true>(p, grid, lds_bytes, s)
                   : launch_tile_b<float, false>(p, grid, lds_bytes, s);
    return vec ? launch_tile_b<double, true>(p, grid, lds_bytes, s)
               : launch_tile_b<double, false>(p, grid, lds_bytes, s);
}

static uint32_t real_grid(const struct fftk_real_params* p)
{
    uint64_t total = (uint64_t)(p->half / 2 + 1) * p->rows0 * p->rows1 * p->rows2;
    return (uint32_t)((total + 255) / 256);
}

int fftrt_launch_real_post(const struct fftk_real_params* p, int precision, void* stream)
{
    uint32_t grid = real_grid(p);
    if(precision == 0)
        {
            if(has_callbacks(p))
                hipLaunchKernelGGL((real_post_kernel<float, true>), dim3(grid), dim3(256), 0, (hipStream_t)stream, *p);
            else
                hipLaunchKernelGGL((real_post_kernel<float, false>), dim3(grid), dim3(256), 0, (hipStream_t)stream, *p);
        }
    else
        {
            if(has_callbacks(p))
                hipLaunchKernelGGL((real_post_kernel<double, true>), dim3(grid), dim3(256), 0, (hipStream_t)stream, *p);
            else
                hipLaunchKernelGGL((real_post_kernel<double, false>), dim3(grid), dim3(256), 0, (hipStream_t)stream, *p);
        }
    return (int)hipGetLastError();
}

int fftrt_launch_callback_copy(const struct fftk_cb_params* p, int precision, int complex_elems, void* stream)
{
    uint64_t total = (uint64_t)p->len[0] * p->len[1] * p->len[2] * p->batch;
    uint64_t grid  = (total + 255) / 256;
    if(grid == 0 || grid >= (1ull << 31))
        return (int)hipErrorInvalidValue;
    hipStream_t s = (hipStream_t)stream;
    dim3        g((uint32_t)grid), b(256);
    if(precision == 0 && complex_elems)
        hipLaunchKernelGGL(callback_copy_kernel<float2>, g, b, 0, s, *p);
    else if(precision == 0)
        hipLaunchKernelGGL(callback_copy_kernel<float>, g, b, 0, s, *p);
    else if(complex_elems)
        hipLaunchKernelGGL(callback_copy_kernel<double2>, g, b, 0, s, *p);
    else
        hipLaunchKernelGGL(callback_copy_kernel<double>, g, b, 0, s, *p);
    return (int)hipGetLastError();
}

int fftrt_launch_half_copy(const struct fftk_cb_params* p, int complex_elems, void* stream)
{
    uint64_t total = (uint64_t)p->len[0] * p->len[1] * p->len[2] * p->batch;
    uint64_t grid  = (total + 255) / 256;
    if(grid == 0 || grid >= (1ull << 31))
        return (int)hipErrorInvalidValue;
    hipStream_t s = (hipStream_t)stream;
    dim3        g((uint32_t)grid), b(256);
    if(complex_elems)
        hipLaunchKernelGGL((half_copy_kernel<fft_half2, float2>), g, b, 0, s, *p);
    else
        hipLaunchKernelGGL((half_copy_kernel<fft_half, float>), g, b, 0, s, *p);
    return (int)hipGetLastError();
}

int fftrt_launch_copy(const struct fftk_copy_params* p, int precision, void* stream)
{
    uint64_t total = (uint64_t)p->cnt * p->rows0 * p->rows1 * p->rows2;
    uint64_t grid  = (total + 255) / 256;
    if(grid == 0 || grid >= (1ull << 31))
        return (int)hipErrorInvalidValue;
    if(precision == 0)
        {
            if(has_callbacks(p))
                hipLaunchKernelGGL((row_copy_kernel<float, true>), dim3((uint32_t)grid), dim3(256), 0, (hipStream_t)stream, *p);
            else
                hipLaunchKernelGGL((row_copy_kernel<float, false>), dim3((uint32_t)grid), dim3(256), 0, (hipStream_t)stream, *p);
        }
    else
        {
            if(has_callbacks(p))
                hipLaunchKernelGGL((row_copy_kernel<double, true>), dim3((uint32_t)grid), dim3(256), 0, (hipStream_t)stream, *p);
            else
                hipLaunchKernelGGL((row_copy_kernel<double, false>), dim3((uint32_t)grid), dim3(256), 0, (hipStream_t)stream, *p);
        }
    return (int)hipGetLastError();
}

int fftrt_launch_real_pre(const struct fftk_real_params* p, int precision, void* stream)
{
    uint32_t grid = real_grid(p);
    if(precision == 0)
        {
            if(has_callbacks(p))
                hipLaunchKernelGGL((real_pre_kernel<float, true>), dim3(grid), dim3(256), 0, (hipStream_t)stream, *p);
            else
                hipLaunchKernelGGL((real_pre_kernel<float, false>), dim3(grid), dim3(256), 0, (hipStream_t)stream, *p);
        }
    else
        {
            if(has_callbacks(p))
                hipLaunchKernelGGL((real_pre_kernel<double, true>), dim3(grid), dim3(256), 0, (hipStream_t)stream, *p);
            else
                hipLaunchKernelGGL((real_pre_kernel<double, false>), dim3(grid), dim3(256), 0, (hipStream_t)stream, *p);
        }
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// Work area of the execute variant that allocates nothing: a file-scope device
// array.  Every device holds its own copy at its own address, so the address is
// looked up once per device (with that device current) and kept; host code never
// passes the array's name to a kernel or a copy, only the looked-up pointer.
static __device__ __align__(256) unsigned char scratch[FFTRT_STATIC_SCRATCH_BYTES];

int fftrt_static_scratch(void** ptr, size_t* bytes)
{
    constexpr int     MAX_DEVICES = 64;
    static std::mutex lock;
    static void*      dev_ptr[MAX_DEVICES]; // zero-initialised: not looked up yet
    *ptr   = nullptr;
    *bytes = 0;
    int dev = 0;
    int rc  = (int)hipGetDevice(&dev);
    if(rc)
        return rc;
    if(dev < 0 || dev >= MAX_DEVICES)
        return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(lock);
    if(!dev_ptr[dev])
    {
        void* p = nullptr;
        rc      = (int)hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if(rc)
            return rc;
        if(!p)
            return (int)hipErrorInvalidSymbol;
        dev_ptr[dev] = p;
    }
    *ptr   = dev_ptr[dev];
    *bytes = FFTRT_STATIC_SCRATCH_BYTES;
    return 0;
}

int fftrt_event_create(void** ev)
{
    return (int)hipEventCreate((hipEvent_t*)ev);
}
int fftrt_event_destroy(void* ev)
{
    return (int)hipEventDestroy((hipEvent_t)ev);
}
int fftrt_event_record(void* ev, void* stream)
{
    return (int)hipEventRecord((hipEvent_t)ev, (hipStream_t)stream);
}
int fftrt_event_elapsed_ms(void* start, void* stop, float* ms)
{
    int rc = (int)hipEventSynchronize((hipEvent_t)stop);
    if(rc)
        return rc;
    return (int)hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop);
}
}
