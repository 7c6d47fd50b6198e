// fast2d_core.h -- a whole small 2D complex transform in one workgroup.
//
// A workgroup owns K neighbouring nA x nB transforms (nA the unit-stride dimension), each a
// contiguous block of nA*nB elements.  Phase 1 loads the rows straight into registers and
// transforms them along the first dimension (schedule CfgA), leaving the tile in LDS in natural
// order; phase 2 transforms the columns of the LDS tile (schedule CfgB, elements one row pitch
// apart) and stores straight from registers.  One pass over memory instead of two.
//
// The reference has the same idea in its generated "2D single" kernels
// (library/src/device/generator/stockham_gen_2d.h); this one is built from the pass helpers of
// fast_core.h.
#ifndef ROCFFT_AMD_FAST2D_CORE_H
#define ROCFFT_AMD_FAST2D_CORE_H

#include "fast_core.h"

template <typename CfgA, typename CfgB>
struct Fast2dShape
{
    static constexpr int nA = CfgA::N, nB = CfgB::N;
    static constexpr int PA = CfgA::PITCH; // LDS elements between rows
    static constexpr int TP = nB * PA;     // LDS elements of one transform
    // threads one transform needs: the larger of the two phases
    static constexpr int T1  = nB * CfgA::TPT;
    static constexpr int T2  = nA * CfgB::TPT;
    static constexpr int TPX = T1 > T2 ? T1 : T2;
};

template <typename T, typename CfgA, typename CfgB>
__device__ __forceinline__ void fast2d_body(const fftk_params& p, typename cplx_of<T>::type* lds)
{
    typedef typename cplx_of<T>::type C;
    typedef Fast2dShape<CfgA, CfgB>   Sh;
    constexpr int                     nA = Sh::nA, nB = Sh::nB, PA = Sh::PA, TP = Sh::TP;
    TileCtx<T>                        c;
    tile_decode<T>(p, blockIdx.x, c);
    const uint32_t tid = threadIdx.x;
    const uint32_t K   = p.W;
    const bool     inv = p.dir > 0;
    const C*       src = reinterpret_cast<const C*>(static_cast<const T*>(p.in0) + c.ibase);
    C*             dst = reinterpret_cast<C*>(static_cast<T*>(p.out0) + c.obase);

    // ---------------------------------------------------------------- phase 1: rows
    {
        constexpr int  LAST   = CfgA::NP - 1;
        constexpr int  R0     = CfgA::radix(0);
        constexpr int  S0     = CfgA::S(0);
        constexpr int  M0     = nA / R0;
        const uint32_t w1     = tid / (uint32_t)CfgA::TPT; // row of the tile: transform k, row b
        const uint32_t tt     = tid % (uint32_t)CfgA::TPT;
        const uint32_t k      = w1 / (uint32_t)nB;
        const uint32_t b      = w1 % (uint32_t)nB;
        const bool     active = w1 < K * (uint32_t)nB;
        const bool     ok     = active && (c.tile0 + k < p.tile_cnt);
        C              r[CfgA::EPT];
        if(ok)
        {
            const C* row = src + (uint64_t)k * p.w_is_c + b * (uint32_t)nA;
#pragma unroll
            for(int s = 0; s < S0; ++s)
#pragma unroll
                for(int kk = 0; kk < R0; ++kk)
                    if(fk_live<CfgA, 0>(tt, s))
                    {
                        C v           = row[tt + s * CfgA::TPT + kk * M0];
                        r[s * R0 + kk] = inv ? c_swap(v) : v;
                    }
        }
        fk_passes_tw<T, CfgA>(p.tw, lds, w1, tt, active, r, false);
        if(CfgA::NP > 1)
            __syncthreads();
        if(active)
            fk_write<T, CfgA, LAST>(lds, w1, tt, r);
    }
    __syncthreads();
    // ---------------------------------------------------------------- phase 2: columns
    {
        typedef FkStrideAddr<PA> Col;
        constexpr int            LAST = CfgB::NP - 1;
        constexpr int            RL   = CfgB::radix(LAST);
        constexpr int            SL   = CfgB::S(LAST);
        constexpr int            CL   = nB / RL;
        const uint32_t           cols = K * (uint32_t)nA; // columns of the tile, lanes run along them
        const uint32_t           c2   = tid % cols;
        const uint32_t           tt   = tid / cols;
        const uint32_t           k    = c2 / (uint32_t)nA;
        const uint32_t           a    = c2 % (uint32_t)nA;
        const bool               active = tt < (uint32_t)CfgB::TPT;
        const bool               ok     = active && (c.tile0 + k < p.tile_cnt);
        const uint32_t           base   = k * (uint32_t)TP + a + (a >> CfgA::PADSHIFT);
        C                        r[CfgB::EPT];
        if(active)
            fk_read<T, CfgB, 0, Col>(lds, base, tt, r);
        fk_passes_tw<T, CfgB, Col>(p.tw2, lds, base, tt, active, r, true);
        if(ok)
        {
            C*      out = dst + (uint64_t)k * p.w_os_c + a;
            const T sc  = (p.flags & FFTK_F_SCALE) ? (T)p.scale : (T)1;
#pragma unroll
            for(int s = 0; s < SL; ++s)
#pragma unroll
                for(int kk = 0; kk < RL; ++kk)
                    if(fk_live<CfgB, LAST>(tt, s))
                    {
                        const uint32_t q = tt + s * CfgB::TPT + kk * CL;
                        C              v = inv ? c_swap(r[s * RL + kk]) : r[s * RL + kk];
                        v.x *= sc;
                        v.y *= sc;
                        out[q * (uint32_t)nA] = v;
                    }
        }
    }
}

#endif
