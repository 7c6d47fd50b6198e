// fast2d_core.h -- a whole small 2D complex transform in one workgroup.
//
// A workgroup owns K neighbouring nA x nB transforms (nA the unit-stride dimension; rows
// p.t_is_c / p.t_os_c complex elements apart on the two sides).  Phase 1 loads the rows straight into registers and
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
            const C* row = src + (uint64_t)k * p.w_is_c + b * p.t_is_c;
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
                        out[q * p.t_os_c] = v;
                    }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Real 2D transforms in one workgroup.  The real dimension has 2L points and is transformed as
// L complex points (CfgA is the schedule of length L) with the even-length post-/pre-processing
// (reference library/src/device/kernels/real2complex_device.h:25-254) done on the LDS tile; the
// tile holds L+1 Hermitian bins per row.

template <typename CfgA, typename CfgB>
struct Fast2dRealShape
{
    static constexpr int L  = CfgA::N, nB = CfgB::N, H = L + 1;
    static constexpr int PH = ((H + (L >> CfgA::PADSHIFT) + 1) | 1); // LDS elements between rows
    static constexpr int TP = nB * PH;
    static constexpr int T1  = nB * CfgA::TPT; // row phase
    static constexpr int T2  = H * CfgB::TPT;  // column phase
    static constexpr int TPX = T1 > T2 ? T1 : T2;
    static __host__ __device__ __forceinline__ uint32_t at(uint32_t row, uint32_t j)
    {
        return row * (uint32_t)PH + j + (j >> CfgA::PADSHIFT);
    }
};

template <typename CfgA, typename Sh>
struct FkRealRowAddr
{
    static FFT_DEV uint32_t at(uint32_t row, uint32_t j)
    {
        return Sh::at(row, j);
    }
};

// real forward: 2L x nB reals -> (L+1) x nB Hermitian bins
template <typename T, typename CfgA, typename CfgB>
__device__ __forceinline__ void fast2d_r2c_body(const fftk_params& p, typename cplx_of<T>::type* lds)
{
    typedef typename cplx_of<T>::type   C;
    typedef Fast2dRealShape<CfgA, CfgB> Sh;
    typedef FkRealRowAddr<CfgA, Sh>     Row;
    typedef FkStrideAddr<Sh::PH>        Col;
    constexpr int                       L = Sh::L, nB = Sh::nB, H = Sh::H, TP = Sh::TP;
    TileCtx<T>                          c;
    tile_decode<T>(p, blockIdx.x, c);
    const uint32_t tid = threadIdx.x;
    const uint32_t K   = p.W;
    const C*       src = reinterpret_cast<const C*>(static_cast<const T*>(p.in0) + c.ibase);
    C*             dst = reinterpret_cast<C*>(static_cast<T*>(p.out0) + c.obase);
    // ---- rows: half-length forward transforms of the real pairs
    {
        constexpr int  LAST   = CfgA::NP - 1;
        constexpr int  R0     = CfgA::radix(0);
        constexpr int  S0     = CfgA::S(0);
        constexpr int  M0     = L / R0;
        const uint32_t w1     = tid / (uint32_t)CfgA::TPT;
        const uint32_t tt     = tid % (uint32_t)CfgA::TPT;
        const uint32_t k      = w1 / (uint32_t)nB;
        const uint32_t b      = w1 % (uint32_t)nB;
        const bool     active = w1 < K * (uint32_t)nB;
        const bool     ok     = active && (c.tile0 + k < p.tile_cnt);
        C              r[CfgA::EPT];
        if(ok)
        {
            const C* row = src + (uint64_t)k * p.w_is_c + b * p.t_is_c;
#pragma unroll
            for(int s = 0; s < S0; ++s)
#pragma unroll
                for(int kk = 0; kk < R0; ++kk)
                    if(fk_live<CfgA, 0>(tt, s))
                        r[s * R0 + kk] = row[tt + s * CfgA::TPT + kk * M0];
        }
        fk_passes_tw<T, CfgA, Row>(p.tw, lds, w1, tt, active, r, false);
        if(CfgA::NP > 1)
            __syncthreads();
        if(active)
            fk_write<T, CfgA, LAST, Row>(lds, w1, tt, r);
    }
    __syncthreads();
    // ---- post-processing in place on the LDS rows: pairs (j, L-j), j = 0..L/2
    {
        constexpr uint32_t PAIRS = L / 2 + 1;
        const C*           htw   = static_cast<const C*>(p.half_tw);
        const uint32_t     items = K * (uint32_t)nB * PAIRS;
        for(uint32_t i = tid; i < items; i += p.nthreads)
        {
            const uint32_t row = i / PAIRS, j = i % PAIRS, jq = (uint32_t)L - j;
            C              zp = lds[Sh::at(row, j)];
            C              o0, o1;
            if(j == 0)
            {
                o0.x = zp.x + zp.y;
                o0.y = 0;
                o1.x = zp.x - zp.y;
                o1.y = 0;
            }
            else
            {
                C zq = lds[Sh::at(row, jq)];
                C t  = htw[j];
                C u, v;
                u.x  = (T)0.5 * (zp.x + zq.x);
                u.y  = (T)0.5 * (zp.y + zq.y);
                v.x  = (T)0.5 * (zp.x - zq.x);
                v.y  = (T)0.5 * (zp.y - zq.y);
                o0.x = u.x + v.x * t.y + u.y * t.x;
                o0.y = v.y + u.y * t.y - v.x * t.x;
                o1.x = u.x - v.x * t.y - u.y * t.x;
                o1.y = -v.y + u.y * t.y - v.x * t.x;
            }
            lds[Sh::at(row, j)]  = o0;
            lds[Sh::at(row, jq)] = o1;
        }
    }
    __syncthreads();
    // ---- columns: forward transforms of the L+1 bin columns
    {
        constexpr int  LAST   = CfgB::NP - 1;
        constexpr int  RL     = CfgB::radix(LAST);
        constexpr int  SL     = CfgB::S(LAST);
        constexpr int  CL     = nB / RL;
        const uint32_t cols   = K * (uint32_t)H;
        const uint32_t c2     = tid % cols;
        const uint32_t tt     = tid / cols;
        const uint32_t k      = c2 / (uint32_t)H;
        const uint32_t a      = c2 % (uint32_t)H;
        const bool     active = tt < (uint32_t)CfgB::TPT;
        const bool     ok     = active && (c.tile0 + k < p.tile_cnt);
        const uint32_t base   = k * (uint32_t)TP + a + (a >> CfgA::PADSHIFT);
        C              r[CfgB::EPT];
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
                        C              v = r[s * RL + kk];
                        v.x *= sc;
                        v.y *= sc;
                        out[q * p.t_os_c] = v;
                    }
        }
    }
}

// real inverse: (L+1) x nB Hermitian bins -> 2L x nB reals
template <typename T, typename CfgA, typename CfgB>
__device__ __forceinline__ void fast2d_c2r_body(const fftk_params& p, typename cplx_of<T>::type* lds)
{
    typedef typename cplx_of<T>::type   C;
    typedef Fast2dRealShape<CfgA, CfgB> Sh;
    typedef FkRealRowAddr<CfgA, Sh>     Row;
    typedef FkStrideAddr<Sh::PH>        Col;
    constexpr int                       L = Sh::L, nB = Sh::nB, H = Sh::H, TP = Sh::TP;
    TileCtx<T>                          c;
    tile_decode<T>(p, blockIdx.x, c);
    const uint32_t tid = threadIdx.x;
    const uint32_t K   = p.W;
    const C*       src = reinterpret_cast<const C*>(static_cast<const T*>(p.in0) + c.ibase);
    C*             dst = reinterpret_cast<C*>(static_cast<T*>(p.out0) + c.obase);
    // ---- columns: inverse transforms of the L+1 bin columns, straight from global memory
    {
        constexpr int  LAST   = CfgB::NP - 1;
        constexpr int  R0     = CfgB::radix(0);
        constexpr int  S0     = CfgB::S(0);
        constexpr int  M0     = nB / R0;
        constexpr int  RL     = CfgB::radix(LAST);
        constexpr int  SL     = CfgB::S(LAST);
        constexpr int  CL     = nB / RL;
        const uint32_t cols   = K * (uint32_t)H;
        const uint32_t c2     = tid % cols;
        const uint32_t tt     = tid / cols;
        const uint32_t k      = c2 / (uint32_t)H;
        const uint32_t a      = c2 % (uint32_t)H;
        const bool     active = tt < (uint32_t)CfgB::TPT;
        const bool     ok     = active && (c.tile0 + k < p.tile_cnt);
        const uint32_t base   = k * (uint32_t)TP + a + (a >> CfgA::PADSHIFT);
        C              r[CfgB::EPT];
        if(ok)
        {
            const C* col = src + (uint64_t)k * p.w_is_c + a;
#pragma unroll
            for(int s = 0; s < S0; ++s)
#pragma unroll
                for(int kk = 0; kk < R0; ++kk)
                    if(fk_live<CfgB, 0>(tt, s))
                        r[s * R0 + kk] = c_swap(col[(tt + s * CfgB::TPT + kk * M0) * p.t_is_c]);
        }
        fk_passes_tw<T, CfgB, Col>(p.tw2, lds, base, tt, active, r, false);
        if(CfgB::NP > 1)
            __syncthreads();
        if(active)
        {
            // natural order, true values (the exchange of re/im undone)
#pragma unroll
            for(int s = 0; s < SL; ++s)
#pragma unroll
                for(int kk = 0; kk < RL; ++kk)
                    if(fk_live<CfgB, LAST>(tt, s))
                        lds[Col::at(base, tt + s * CfgB::TPT + kk * CL)] = c_swap(r[s * RL + kk]);
        }
    }
    __syncthreads();
    // ---- pre-processing in place on the LDS rows: bins (j, L-j) -> half-length input (j, L-j)
    {
        constexpr uint32_t PAIRS = L / 2 + 1;
        const C*           htw   = static_cast<const C*>(p.half_tw);
        const uint32_t     items = K * (uint32_t)nB * PAIRS;
        for(uint32_t i = tid; i < items; i += p.nthreads)
        {
            const uint32_t row = i / PAIRS, j = i % PAIRS, jq = (uint32_t)L - j;
            C              a  = lds[Sh::at(row, j)];
            C              bq = lds[Sh::at(row, jq)];
            C              zj, zq;
            if(j == 0)
            {
                // only the real parts of bins 0 and L count
                zj.x = a.x + bq.x;
                zj.y = a.x - bq.x;
                zq   = zj;
            }
            else
            {
                C t  = htw[j];
                C u  = c_add(a, bq);
                C v  = c_sub(a, bq);
                zj.x = u.x + v.x * t.y - u.y * t.x;
                zj.y = v.y + u.y * t.y + v.x * t.x;
                zq.x = u.x - v.x * t.y + u.y * t.x;
                zq.y = -v.y + u.y * t.y + v.x * t.x;
            }
            if(j != 0)
                lds[Sh::at(row, jq)] = zq;
            lds[Sh::at(row, j)] = zj;
        }
    }
    __syncthreads();
    // ---- rows: half-length inverse transforms, stored as real pairs
    {
        constexpr int  LAST   = CfgA::NP - 1;
        constexpr int  RL     = CfgA::radix(LAST);
        constexpr int  SL     = CfgA::S(LAST);
        constexpr int  CL     = L / RL;
        constexpr int  R0     = CfgA::radix(0);
        constexpr int  S0     = CfgA::S(0);
        const uint32_t w1     = tid / (uint32_t)CfgA::TPT;
        const uint32_t tt     = tid % (uint32_t)CfgA::TPT;
        const uint32_t k      = w1 / (uint32_t)nB;
        const uint32_t b      = w1 % (uint32_t)nB;
        const bool     active = w1 < K * (uint32_t)nB;
        const bool     ok     = active && (c.tile0 + k < p.tile_cnt);
        C              r[CfgA::EPT];
        if(active)
        {
            fk_read<T, CfgA, 0, Row>(lds, w1, tt, r);
#pragma unroll
            for(int i = 0; i < S0 * R0; ++i)
                r[i] = c_swap(r[i]);
        }
        fk_passes_tw<T, CfgA, Row>(p.tw, lds, w1, tt, active, r, true);
        if(ok)
        {
            C*      row = dst + (uint64_t)k * p.w_os_c + b * p.t_os_c;
            const T sc  = (p.flags & FFTK_F_SCALE) ? (T)p.scale : (T)1;
#pragma unroll
            for(int s = 0; s < SL; ++s)
#pragma unroll
                for(int kk = 0; kk < RL; ++kk)
                    if(fk_live<CfgA, LAST>(tt, s))
                    {
                        C v = c_swap(r[s * RL + kk]);
                        v.x *= sc;
                        v.y *= sc;
                        row[tt + s * CfgA::TPT + kk * CL] = v;
                    }
        }
    }
}

#endif
