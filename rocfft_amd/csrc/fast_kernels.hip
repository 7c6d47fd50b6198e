// fast_kernels.hip -- instantiations of the compile-time-schedule tile kernel
// (fast_core.h) for the power-of-two lengths, and their registry.
#include "fast_core.h"
#include "gpu_rt.h"
#include <hip/hip_runtime.h>
#include <mutex>

namespace
{

// MODE 0: scalar accesses, every fused operation; 1: vector accesses, every fused operation;
// 2: the lean path (vector accesses, interleaved complex on both sides)
// workgroups have up to 256 threads, or 512 when one transform alone needs more than 256
template <typename Cfg>
constexpr int fast_block_limit()
{
    return Cfg::TPT > 256 ? 512 : 256;
}

template <typename T, typename Cfg, int MODE>
__global__ __launch_bounds__(fast_block_limit<Cfg>()) void fast_tile_kernel(const fftk_params p)
{
    typedef typename cplx_of<T>::type C;
    extern __shared__ double2         smem_raw[];
    fast_tile_body<T, Cfg, MODE != 0, MODE == 2>(p, reinterpret_cast<C*>(smem_raw));
}

typedef int (*fast_launch_fn)(const fftk_params*, uint32_t, size_t, hipStream_t);

template <typename T, typename Cfg, int MODE>
int launch_fast(const fftk_params* p, uint32_t grid, size_t lds_bytes, hipStream_t stream)
{
    auto kernel = fast_tile_kernel<T, Cfg, MODE>;
    if(lds_bytes > 64 * 1024)
    {
        static std::once_flag once[16];
        int                   dev = 0;
        (void)hipGetDevice(&dev);
        int rc = 0;
        std::call_once(once[dev & 15], [&]() {
            rc = (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        });
        if(rc)
            return rc;
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(p->nthreads), lds_bytes, stream, *p);
    return (int)hipGetLastError();
}

struct FastEntry
{
    int            precision;
    uint32_t       n;
    uint32_t       radix[4];
    uint32_t       tpt;
    fast_launch_fn lean, vec, scalar;
};

#define FAST_ONE(T, P, N, A, B, C, D)                                                              \
    {P, N, {A, B, C, D}, FastCfg<N, A, B, C, D>::TPT, &launch_fast<T, FastCfg<N, A, B, C, D>, 2>,  \
     &launch_fast<T, FastCfg<N, A, B, C, D>, 1>, &launch_fast<T, FastCfg<N, A, B, C, D>, 0>},
#define FAST_BOTH(N, A, B, C, D) FAST_ONE(float, 0, N, A, B, C, D) FAST_ONE(double, 1, N, A, B, C, D)

// the schedules the planner's factorisation produces for powers of two
const FastEntry g_fast[] = {
    FAST_BOTH(2, 2, 1, 1, 1)
    FAST_BOTH(4, 4, 1, 1, 1)
    FAST_BOTH(8, 8, 1, 1, 1)
    FAST_BOTH(16, 16, 1, 1, 1)
    FAST_BOTH(32, 8, 4, 1, 1)
    FAST_BOTH(64, 16, 4, 1, 1)
    FAST_BOTH(128, 16, 8, 1, 1)
    FAST_BOTH(256, 16, 16, 1, 1)
    FAST_BOTH(512, 16, 8, 4, 1)
    FAST_BOTH(1024, 16, 16, 4, 1)
    FAST_BOTH(2048, 16, 16, 8, 1)
    FAST_BOTH(4096, 16, 16, 16, 1)
    FAST_BOTH(8192, 16, 16, 8, 4)
};

const FastEntry* find_fast(int precision, uint32_t n, const uint32_t* radix, uint32_t nf)
{
    if(nf < 1 || nf > 4)
        return nullptr;
    for(const FastEntry& e : g_fast)
    {
        if(e.precision != precision || e.n != n)
            continue;
        bool same = true;
        for(uint32_t i = 0; i < 4; ++i)
            same = same && e.radix[i] == (i < nf ? radix[i] : 1u);
        if(same)
            return &e;
    }
    return nullptr;
}

} // namespace

extern "C" uint32_t fftrt_fast_tpt(int precision, uint32_t n, const uint32_t* radix, uint32_t nf)
{
    const FastEntry* e = find_fast(precision, n, radix, nf);
    return e ? e->tpt : 0;
}

// called by fftrt_launch_tile (kernels.hip) when the plan asked for the fast kernel
extern "C" int fftrt_launch_fast_tile(const struct fftk_params* p, int precision, int vec, uint32_t grid,
                                      size_t lds_bytes, void* stream)
{
    const FastEntry* e = find_fast(precision, p->n, p->radix, p->nf);
    if(!e || p->T != e->tpt || p->nthreads > (e->tpt > 256 ? 512u : 256u) || p->padshift != 4)
        return (int)hipErrorInvalidValue;
    fast_launch_fn fn = (vec && p->lean) ? e->lean : vec ? e->vec : e->scalar;
    return fn(p, grid, lds_bytes, (hipStream_t)stream);
}
