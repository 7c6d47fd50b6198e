// gpu_rt_emu.cpp -- TEST INFRASTRUCTURE ONLY.
//
// A host implementation of the C-ABI runtime layer (rocfft_amd/csrc/gpu_rt.h):
// "device" memory is host memory and a kernel launch is a loop over workgroups
// and threads that calls the very same phase functions the HIP kernels call
// (rocfft_amd/csrc/tile_core.h), with the barriers replaced by loop boundaries.
// Linked with the planner and API sources it gives librocfft_amd_emu.so, which
// lets the CPU test-suite check the planner's pass lists, strides and fused
// operations numerically without a GPU.  The product library never contains or
// loads this file.
#include "gpu_rt.h"
#include "fast_core.h"
#include "tile_core.h"
#include <cstdlib>
#include <cstring>
#include <vector>

namespace
{
template <typename T>
void emu_passes(const fftk_params& p, typename cplx_of<T>::type* lds)
{
    typedef typename cplx_of<T>::type C;
    std::vector<C>                    regs((size_t)p.nthreads * FFTK_REG_ELEMS);
    for(uint32_t pass = 0; pass < p.nf; ++pass)
    {
        for(int phase = 0; phase < 2; ++phase)
            for(uint32_t tid = 0; tid < p.nthreads; ++tid)
            {
                uint32_t w, tt;
                bool     active;
                thread_role(p, tid, w, tt, active);
                C* r = regs.data() + (size_t)tid * FFTK_REG_ELEMS;
                switch(p.radix[pass])
                {
#define EMU_CASE(R)                                                  \
    case R:                                                          \
        if(phase == 0)                                               \
            pass_read<T, R>(p, lds, w, tt, active, r);               \
        else                                                         \
            pass_write<T, R>(p, (int)pass, lds, w, tt, active, r);   \
        break;
                    EMU_CASE(2)
                    EMU_CASE(3)
                    EMU_CASE(4)
                    EMU_CASE(5)
                    EMU_CASE(6)
                    EMU_CASE(7)
                    EMU_CASE(8)
                    EMU_CASE(9)
                    EMU_CASE(10)
                    EMU_CASE(11)
                    EMU_CASE(12)
                    EMU_CASE(13)
                    EMU_CASE(14)
                    EMU_CASE(15)
                    EMU_CASE(16)
                    EMU_CASE(17)
#undef EMU_CASE
                default:
                    break;
                }
            }
    }
}

template <typename T, bool VEC>
void emu_tile(const fftk_params& p, uint32_t grid, size_t lds_bytes)
{
    typedef typename cplx_of<T>::type C;
    std::vector<C>                    lds(lds_bytes / sizeof(C) + 1);
    for(uint32_t bid = 0; bid < grid; ++bid)
    {
        // poison the LDS so that reads of unwritten slots show up
        for(C& v : lds)
        {
            v.x = (T)1e30;
            v.y = (T)-1e30;
        }
        TileCtx<T> c;
        tile_decode<T>(p, bid, c);
        for(uint32_t tid = 0; tid < p.nthreads; ++tid)
            tile_load<T, VEC>(p, c, lds.data(), tid);
        emu_passes<T>(p, lds.data());
        if(p.flags & FFTK_F_CONV)
        {
            for(uint32_t tid = 0; tid < p.nthreads; ++tid)
                tile_conv<T>(p, c, lds.data(), tid);
            emu_passes<T>(p, lds.data());
        }
        for(uint32_t tid = 0; tid < p.nthreads; ++tid)
            tile_store<T, VEC>(p, c, lds.data(), tid);
    }
}
} // namespace

extern "C" {

int fftrt_device_count(int* count)
{
    *count = 1;
    return 0;
}
int fftrt_device_info(int* device, int* compute_units, int* lds_bytes, char* arch, size_t arch_len)
{
    if(device)
        *device = 0;
    if(compute_units)
        *compute_units = 256;
    if(lds_bytes)
        *lds_bytes = 160 * 1024;
    if(arch && arch_len)
    {
        strncpy(arch, "host-emulation", arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    return 0;
}
static long g_malloc_calls = 0;
// (tests) device allocations made so far
__attribute__((visibility("default"))) long fftrt_emu_malloc_calls(void)
{
    return g_malloc_calls;
}
int fftrt_malloc(void** ptr, size_t bytes)
{
    ++g_malloc_calls;
    *ptr = malloc(bytes ? bytes : 1);
    return *ptr ? 0 : 2;
}
int fftrt_free(void* ptr)
{
    free(ptr);
    return 0;
}
int fftrt_upload(void* dst, const void* src, size_t bytes)
{
    memcpy(dst, src, bytes);
    return 0;
}
int fftrt_download(void* dst, const void* src, size_t bytes)
{
    memcpy(dst, src, bytes);
    return 0;
}
int fftrt_stream_sync(void*)
{
    return 0;
}
int fftrt_device_sync(void)
{
    return 0;
}
int fftrt_stream_capturing(void*)
{
    return 0;
}

// The emulation only has the generic kernel, but it reports the pass schedules of the
// compile-time-schedule kernels, so that the planner makes the same plans as on the GPU and
// the generic kernel gets exercised on those schedules.
namespace
{
struct EmuSched
{
    uint32_t n, radix[4], tpt[2]; // threads per transform in single, double precision
};
#define FAST_SCHED(SLICE, FULL, N, A, B, C, D, TTF, TTD, DBL) \
    {N, {A, B, C, D}, {(uint32_t)FastCfg<N, A, B, C, D, TTF>::TPT, (DBL) ? (uint32_t)FastCfg<N, A, B, C, D, TTD>::TPT : 0u}},
const EmuSched g_sched[] = {
#include "fast_schedules.h"
};
#undef FAST_SCHED
} // namespace

uint32_t fftrt_fast_schedule(int precision, uint32_t n, uint32_t* radix, uint32_t* nf)
{
    for(const EmuSched& e : g_sched)
    {
        if(e.n != n)
            continue;
        uint32_t cnt = 0;
        for(uint32_t i = 0; i < 4; ++i)
            if(e.radix[i] > 1)
                radix[cnt++] = e.radix[i];
        *nf = cnt;
        return e.tpt[precision ? 1 : 0];
    }
    return 0;
}

// the emulation converts half-precision arrays in separate passes
int fftrt_fast_takes_half(uint32_t)
{
    return 0;
}

int fftrt_launch_tile(const struct fftk_params* p, int precision, int vec, uint32_t grid,
                      size_t lds_bytes, void*)
{
    if(p->nthreads == 0 || p->nthreads > 1024 || (p->nthreads & 63) || lds_bytes > 160 * 1024
       || grid == 0)
        return 1;
    if(precision == 0)
        vec ? emu_tile<float, true>(*p, grid, lds_bytes) : emu_tile<float, false>(*p, grid, lds_bytes);
    else
        vec ? emu_tile<double, true>(*p, grid, lds_bytes)
            : emu_tile<double, false>(*p, grid, lds_bytes);
    return 0;
}

int fftrt_launch_real_post(const struct fftk_real_params* p, int precision, void*)
{
    uint64_t total = (uint64_t)(p->half / 2 + 1) * p->rows0 * p->rows1 * p->rows2;
    for(uint64_t g = 0; g < total; ++g)
        precision ? real_post_elem<double>(*p, g) : real_post_elem<float>(*p, g);
    return 0;
}
int fftrt_launch_real_pre(const struct fftk_real_params* p, int precision, void*)
{
    uint64_t total = (uint64_t)(p->half / 2 + 1) * p->rows0 * p->rows1 * p->rows2;
    for(uint64_t g = 0; g < total; ++g)
        precision ? real_pre_elem<double>(*p, g) : real_pre_elem<float>(*p, g);
    return 0;
}

int fftrt_launch_copy(const struct fftk_copy_params* p, int precision, void*)
{
    uint64_t total = (uint64_t)p->cnt * p->rows0 * p->rows1 * p->rows2;
    for(uint64_t g = 0; g < total; ++g)
        precision ? copy_elem<double>(*p, g) : copy_elem<float>(*p, g);
    return 0;
}

int fftrt_launch_callback_copy(const struct fftk_cb_params* p, int precision, int complex_elems, void*)
{
    uint64_t total = (uint64_t)p->len[0] * p->len[1] * p->len[2] * p->batch;
    for(uint64_t g = 0; g < total; ++g)
    {
        if(precision == 0 && complex_elems)
            callback_elem<float2>(*p, g);
        else if(precision == 0)
            callback_elem<float>(*p, g);
        else if(complex_elems)
            callback_elem<double2>(*p, g);
        else
            callback_elem<double>(*p, g);
    }
    return 0;
}

int fftrt_launch_half_copy(const struct fftk_cb_params* p, int complex_elems, void*)
{
    uint64_t total = (uint64_t)p->len[0] * p->len[1] * p->len[2] * p->batch;
    for(uint64_t g = 0; g < total; ++g)
    {
        if(complex_elems)
            half_stage_elem<fft_half2, float2>(*p, g);
        else
            half_stage_elem<fft_half, float>(*p, g);
    }
    return 0;
}

// no one-workgroup 2D kernel in the emulation: such plans take the per-dimension passes here
int fftrt_fast2d_info(uint32_t, uint32_t, uint32_t*, uint32_t*, uint32_t*, uint32_t*, uint32_t*, uint32_t*,
                      uint32_t*)
{
    return 0;
}
int fftrt_launch_fast2d(const struct fftk_params*, int, uint32_t, size_t, void*)
{
    return 1;
}
int fftrt_fast2d_real_info(uint32_t, uint32_t, uint32_t*, uint32_t*, uint32_t*, uint32_t*, uint32_t*, uint32_t*,
                           uint32_t*)
{
    return 0;
}
int fftrt_launch_fast2d_real(const struct fftk_params*, int, int, uint32_t, size_t, void*)
{
    return 1;
}

int fftrt_has_big32k(void)
{
    return 0;
}
int fftrt_launch_big32k(const struct fftk_big_params*, void*)
{
    return 1;
}

int fftrt_static_scratch(void** ptr, size_t* bytes)
{
    static std::vector<unsigned char> area(FFTRT_STATIC_SCRATCH_BYTES);
    *ptr   = area.data();
    *bytes = area.size();
    return 0;
}
int fftrt_copy_probe(const struct rocfft_amd_probe*, void*)
{
    return 1; // measurement only: nothing to time without a device
}
int fftrt_event_create(void** ev)
{
    *ev = nullptr;
    return 0;
}
int fftrt_event_destroy(void*)
{
    return 0;
}
int fftrt_event_record(void*, void*)
{
    return 0;
}
int fftrt_event_elapsed_ms(void*, void*, float* ms)
{
    *ms = 0;
    return 0;
}
}
