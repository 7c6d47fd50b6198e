// TEST INFRASTRUCTURE: load/store callbacks with the signatures of the reference API
// (library/include/rocfft/rocfft.h:533-612), compiled once for the host emulation and once
// as device functions.  The load callback multiplies every element by the scalar cbdata
// points to; the store callback multiplies by its scalar before writing.
#ifndef ROCFFT_AMD_TEST_CB_FUNCS_H
#define ROCFFT_AMD_TEST_CB_FUNCS_H
#include <stddef.h>

#ifdef __HIPCC__
#include <hip/hip_runtime.h>
#define CB_FN __device__
#else
#define CB_FN
struct float2
{
    float x, y;
};
struct double2
{
    double x, y;
};
#endif

template <typename S>
CB_FN S cb_load_real(S* data, size_t offset, void* cbdata, void*)
{
    return data[offset] * *static_cast<const S*>(cbdata);
}
template <typename E, typename S>
CB_FN E cb_load_cplx(E* data, size_t offset, void* cbdata, void*)
{
    E       v = data[offset];
    const S s = *static_cast<const S*>(cbdata);
    v.x *= s;
    v.y *= s;
    return v;
}
template <typename S>
CB_FN void cb_store_real(S* data, size_t offset, S element, void* cbdata, void*)
{
    data[offset] = element * *static_cast<const S*>(cbdata);
}
template <typename E, typename S>
CB_FN void cb_store_cplx(E* data, size_t offset, E element, void* cbdata, void*)
{
    const S s = *static_cast<const S*>(cbdata);
    element.x *= s;
    element.y *= s;
    data[offset] = element;
}
#endif
