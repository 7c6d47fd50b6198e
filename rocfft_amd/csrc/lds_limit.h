// lds_limit.h -- raising a kernel's dynamic-LDS limit above the 64 KB default.
//
// hipFuncSetAttribute is needed once per kernel and device before a launch may ask for more
// than 64 KB of dynamic LDS.  The state is kept per kernel (one FftLdsLimit per template
// instantiation, as a function-local static of its launcher) and per device: a failed
// attempt is reported to its caller and tried again by the next launch, so no launch goes
// ahead with the limit unraised.  Not a stream operation: legal during graph capture.
#ifndef ROCFFT_AMD_LDS_LIMIT_H
#define ROCFFT_AMD_LDS_LIMIT_H

#include <atomic>
#include <hip/hip_runtime.h>

struct FftLdsLimit
{
    static constexpr int MAX_DEVICES = 64;
    std::atomic<int>     raised[MAX_DEVICES]; // zero-initialised as a static
    // 0 on success, else the HIP error code
    template <typename K>
    int allow(K kernel, int bytes = 160 * 1024)
    {
        int dev = 0;
        int rc  = (int)hipGetDevice(&dev);
        if(rc)
            return rc;
        if(dev < 0 || dev >= MAX_DEVICES)
            return (int)hipErrorInvalidDevice;
        if(raised[dev].load(std::memory_order_acquire))
            return 0;
        rc = (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if(rc == 0)
            raised[dev].store(1, std::memory_order_release);
        return rc;
    }
};

#endif
