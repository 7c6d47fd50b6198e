// TEST INFRASTRUCTURE: host builds of the test callbacks, for the host emulation of the runtime.
#include "cb_funcs.h"

// which: 0 load, 1 store; complex_elems: 0 real, 1 complex; precision: 0 single, 1 double
extern "C" void* cb_get(int which, int complex_elems, int precision)
{
    if(which == 0)
    {
        if(complex_elems)
            return precision ? (void*)&cb_load_cplx<double2, double> : (void*)&cb_load_cplx<float2, float>;
        return precision ? (void*)&cb_load_real<double> : (void*)&cb_load_real<float>;
    }
    if(complex_elems)
        return precision ? (void*)&cb_store_cplx<double2, double> : (void*)&cb_store_cplx<float2, float>;
    return precision ? (void*)&cb_store_real<double> : (void*)&cb_store_real<float>;
}
