// fast2d_kernels.hip -- instantiations of the one-workgroup 2D kernel (fast2d_core.h) for the
// power-of-two sizes 8..64 in each dimension, and their registry.
#include "fast2d_core.h"
#include "gpu_rt.h"
#include <hip/hip_runtime.h>

namespace
{

// schedules of the four lengths (the same as the 1D compiled kernels of these lengths)
typedef FastCfg<4, 4, 1, 1, 1>   C4;
typedef FastCfg<8, 8, 1, 1, 1>   C8;
typedef FastCfg<16, 16, 1, 1, 1> C16;
typedef FastCfg<32, 8, 4, 1, 1>  C32;
typedef FastCfg<64, 16, 4, 1, 1> C64;

template <typename T, typename CfgA, typename CfgB>
__global__ __launch_bounds__(512) void fast2d_kernel(const fftk_params p)
{
    typedef typename cplx_of<T>::type C;
    extern __shared__ double2         smem_raw[];
    fast2d_body<T, CfgA, CfgB>(p, reinterpret_cast<C*>(smem_raw));
}

// MODE 1: real forward, 2: real inverse (CfgA is the schedule of half the real length)
template <typename T, typename CfgA, typename CfgB, int MODE>
__global__ __launch_bounds__(512) void fast2d_real_kernel(const fftk_params p)
{
    typedef typename cplx_of<T>::type C;
    extern __shared__ double2         smem_raw[];
    if(MODE == 1)
        fast2d_r2c_body<T, CfgA, CfgB>(p, reinterpret_cast<C*>(smem_raw));
    else
        fast2d_c2r_body<T, CfgA, CfgB>(p, reinterpret_cast<C*>(smem_raw));
}

typedef int (*launch2d_fn)(const fftk_params*, uint32_t, size_t, hipStream_t);

template <typename T, typename CfgA, typename CfgB, int MODE>
int launch2d_real(const fftk_params* p, uint32_t grid, size_t lds_bytes, hipStream_t stream)
{
    hipLaunchKernelGGL((fast2d_real_kernel<T, CfgA, CfgB, MODE>), dim3(grid), dim3(p->nthreads), lds_bytes, stream,
                       *p);
    return (int)hipGetLastError();
}

template <typename T, typename CfgA, typename CfgB>
int launch2d(const fftk_params* p, uint32_t grid, size_t lds_bytes, hipStream_t stream)
{
    hipLaunchKernelGGL((fast2d_kernel<T, CfgA, CfgB>), dim3(grid), dim3(p->nthreads), lds_bytes, stream, *p);
    return (int)hipGetLastError();
}

struct Entry2d
{
    uint32_t    nA, nB, tptA, tptB, pitchA;
    uint32_t    radixA[4], radixB[4];
    launch2d_fn f32, f64;
};

#define E2D(A, B)                                                                                    \
    {A::N, B::N, A::TPT, B::TPT, A::PITCH, {A::R0, A::R1, A::R2, A::R3}, {B::R0, B::R1, B::R2, B::R3}, \
     &launch2d<float, A, B>, &launch2d<double, A, B>},
#define E2D_ROW(A) E2D(A, C8) E2D(A, C16) E2D(A, C32) E2D(A, C64)

const Entry2d g_2d[] = {E2D_ROW(C8) E2D_ROW(C16) E2D_ROW(C32) E2D_ROW(C64)};

const Entry2d* find2d(uint32_t nA, uint32_t nB)
{
    for(const Entry2d& e : g_2d)
        if(e.nA == nA && e.nB == nB)
            return &e;
    return nullptr;
}

// real transforms: 2L x nB, L = 4..32
struct Entry2dReal
{
    uint32_t    L, nB, tptA, tptB, pitch;
    uint32_t    radixA[4], radixB[4];
    launch2d_fn fwd32, fwd64, inv32, inv64;
};
#define E2R(A, B)                                                                                             \
    {A::N, B::N, A::TPT, B::TPT, (uint32_t)Fast2dRealShape<A, B>::PH, {A::R0, A::R1, A::R2, A::R3},           \
     {B::R0, B::R1, B::R2, B::R3}, &launch2d_real<float, A, B, 1>, &launch2d_real<double, A, B, 1>,           \
     &launch2d_real<float, A, B, 2>, &launch2d_real<double, A, B, 2>},
#define E2R_ROW(A) E2R(A, C8) E2R(A, C16) E2R(A, C32) E2R(A, C64)
const Entry2dReal g_2dr[] = {E2R_ROW(C4) E2R_ROW(C8) E2R_ROW(C16) E2R_ROW(C32)};

const Entry2dReal* find2dr(uint32_t L, uint32_t nB)
{
    for(const Entry2dReal& e : g_2dr)
        if(e.L == L && e.nB == nB)
            return &e;
    return nullptr;
}

} // namespace

extern "C" int fftrt_fast2d_real_info(uint32_t L, uint32_t nB, uint32_t* radixA, uint32_t* nfA, uint32_t* radixB,
                                      uint32_t* nfB, uint32_t* tptA, uint32_t* tptB, uint32_t* pitch)
{
    const Entry2dReal* e = find2dr(L, nB);
    if(!e)
        return 0;
    uint32_t ca = 0, cb = 0;
    for(int i = 0; i < 4; ++i)
    {
        if(e->radixA[i] > 1)
            radixA[ca++] = e->radixA[i];
        if(e->radixB[i] > 1)
            radixB[cb++] = e->radixB[i];
    }
    *nfA   = ca;
    *nfB   = cb;
    *tptA  = e->tptA;
    *tptB  = e->tptB;
    *pitch = e->pitch;
    return 1;
}

extern "C" int fftrt_launch_fast2d_real(const struct fftk_params* p, int precision, int inverse, uint32_t grid,
                                        size_t lds_bytes, void* stream)
{
    const Entry2dReal* e = find2dr(p->n, p->n2);
    if(!e || p->nthreads == 0 || p->nthreads > 512 || (p->nthreads & 63) || lds_bytes > 64 * 1024 || grid == 0)
        return (int)hipErrorInvalidValue;
    launch2d_fn fn = inverse ? (precision ? e->inv64 : e->inv32) : (precision ? e->fwd64 : e->fwd32);
    return fn(p, grid, lds_bytes, (hipStream_t)stream);
}

extern "C" int fftrt_fast2d_info(uint32_t nA, uint32_t nB, uint32_t* radixA, uint32_t* nfA, uint32_t* radixB,
                                 uint32_t* nfB, uint32_t* tptA, uint32_t* tptB, uint32_t* pitchA)
{
    const Entry2d* e = find2d(nA, nB);
    if(!e)
        return 0;
    uint32_t ca = 0, cb = 0;
    for(int i = 0; i < 4; ++i)
    {
        if(e->radixA[i] > 1)
            radixA[ca++] = e->radixA[i];
        if(e->radixB[i] > 1)
            radixB[cb++] = e->radixB[i];
    }
    *nfA    = ca;
    *nfB    = cb;
    *tptA   = e->tptA;
    *tptB   = e->tptB;
    *pitchA = e->pitchA;
    return 1;
}

extern "C" int fftrt_launch_fast2d(const struct fftk_params* p, int precision, uint32_t grid, size_t lds_bytes,
                                   void* stream)
{
    const Entry2d* e = find2d(p->n, p->n2);
    if(!e || p->nthreads == 0 || p->nthreads > 512 || (p->nthreads & 63) || lds_bytes > 64 * 1024 || grid == 0)
        return (int)hipErrorInvalidValue;
    return (precision ? e->f64 : e->f32)(p, grid, lds_bytes, (hipStream_t)stream);
}
