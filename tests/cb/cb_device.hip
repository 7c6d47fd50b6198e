// TEST INFRASTRUCTURE: device builds of the test callbacks.  Device function addresses are taken
// on the device (a __device__ variable initialised with the address) and read back, which is how
// users of the reference obtain the pointers they pass to rocfft_execution_info_set_*_callback.
#include "cb_funcs.h"
#include <hip/hip_runtime.h>

__device__ void* g_cb_table[8] = {(void*)&cb_load_real<float>,
                                  (void*)&cb_load_real<double>,
                                  (void*)&cb_load_cplx<float2, float>,
                                  (void*)&cb_load_cplx<double2, double>,
                                  (void*)&cb_store_real<float>,
                                  (void*)&cb_store_real<double>,
                                  (void*)&cb_store_cplx<float2, float>,
                                  (void*)&cb_store_cplx<double2, double>};

extern "C" void* cb_get(int which, int complex_elems, int precision)
{
    void* table[8] = {nullptr};
    if(hipMemcpyFromSymbol(table, HIP_SYMBOL(g_cb_table), sizeof(table)) != hipSuccess)
        return nullptr;
    return table[(which ? 4 : 0) + (complex_elems ? 2 : 0) + (precision ? 1 : 0)];
}
