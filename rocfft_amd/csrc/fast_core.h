// fast_core.h -- tile FFT kernel with a compile-time pass schedule.
//
// Same tile model as tile_core.h (a workgroup owns W transforms of length N),
// but length, radices and threads per transform are template parameters, every
// thread keeps its (at most FFTK_REG_ELEMS) elements in registers for the whole kernel,
// and -- where the lane order matches the fast axis in memory -- the first pass
// loads straight from global memory into registers and the last pass stores
// straight from registers, so LDS is only used for the exchanges between passes.
// When the lane order does not match (row-in/column-out passes) or the fused
// operation needs partner elements (real pre/post-processing), that side is
// staged through LDS with tile_load / tile_store of tile_core.h.
//
// The reference reaches the same effect with generated kernels
// ("direct to/from register", library/src/device/generator/stockham_gen_base.h:287-300,
// :823-913); this is a hand-written template, not generated code.
#ifndef ROCFFT_AMD_FAST_CORE_H
#define ROCFFT_AMD_FAST_CORE_H

#include "tile_core.h"

// TPT_ = 0 takes the fewest threads per transform that the register budget allows; a larger
// value spreads a transform over more lanes (longer contiguous runs per access, fewer
// registers per thread).
template <int N_, int R0_, int R1_, int R2_, int R3_, int TPT_ = 0>
struct FastCfg
{
    static constexpr int N  = N_;
    static constexpr int R0 = R0_, R1 = R1_, R2 = R2_, R3 = R3_;
    static constexpr int NP = (R0_ > 1) + (R1_ > 1) + (R2_ > 1) + (R3_ > 1);
    static constexpr int max2(int a, int b)
    {
        return a > b ? a : b;
    }
    static constexpr int radix(int p)
    {
        return p == 0 ? R0_ : p == 1 ? R1_ : p == 2 ? R2_ : R3_;
    }
    // threads one pass of radix r needs when a thread holds at most FFTK_REG_ELEMS values:
    // the same rule the planner applies to the generic kernel
    static constexpr int need(int r)
    {
        return r > 1 ? (N_ / r + FFTK_REG_ELEMS / r - 1) / (FFTK_REG_ELEMS / r) : 1;
    }
    static constexpr int TPT_MIN = max2(max2(need(R0_), need(R1_)), max2(need(R2_), need(R3_)));
    static constexpr int TPT     = TPT_ ? TPT_ : TPT_MIN; // threads per transform
    static_assert(TPT >= TPT_MIN, "too few threads per transform for the register budget");
    // butterflies a thread computes in pass p; when N/radix is no multiple of TPT the
    // last slot of the higher lanes is idle (live() tells)
    static constexpr int S(int p)
    {
        return (N_ / radix(p) + TPT - 1) / TPT;
    }
    static constexpr bool exact(int p)
    {
        return (N_ / radix(p)) % TPT == 0;
    }
    static constexpr int elems(int p)
    {
        return p < NP ? S(p) * radix(p) : 0;
    }
    static constexpr int EPT = max2(max2(elems(0), elems(1)), max2(elems(2), elems(3))); // register elements per thread
    static constexpr int cum(int p)
    {
        return p == 0 ? 1 : p == 1 ? R0_ : p == 2 ? R0_ * R1_ : R0_ * R1_ * R2_;
    }
    static constexpr int twoff(int p)
    {
        // offset of pass p in the stacked twiddle table: sum over 1 <= q < p of cum(q)*(radix(q)-1)
        return p <= 1 ? 0 : twoff(p - 1) + cum(p - 1) * (radix(p - 1) - 1);
    }
    static constexpr int PADSHIFT = 4;
    static constexpr int PITCH    = (N_ + ((N_ - 1) >> PADSHIFT) + 1) | 1;
    static_assert(N_ == R0_ * R1_ * R2_ * R3_, "radices must multiply to N");
    static_assert(EPT <= FFTK_REG_ELEMS, "a thread holds at most FFTK_REG_ELEMS values");
};

template <typename Cfg>
FFT_DEV uint32_t fk_addr(uint32_t w, uint32_t j)
{
    return w * Cfg::PITCH + j + (j >> Cfg::PADSHIFT);
}

// does lane tt have a butterfly in slot s of pass P?
template <typename Cfg, int P>
FFT_DEV bool fk_live(uint32_t tt, int s)
{
    return Cfg::exact(P) || tt + (uint32_t)(s * Cfg::TPT) < (uint32_t)(Cfg::N / Cfg::radix(P));
}

// position of element (butterfly slot s, input k) of pass P held by lane tt
template <typename Cfg, int P>
FFT_DEV uint32_t fk_in_pos(uint32_t tt, int s, int k)
{
    constexpr int R = Cfg::radix(P);
    return tt + s * Cfg::TPT + k * (Cfg::N / R);
}

template <typename Cfg, int P>
FFT_DEV uint32_t fk_out_pos(uint32_t tt, int s, int k)
{
    constexpr int      R = Cfg::radix(P);
    constexpr uint32_t c = Cfg::cum(P);
    uint32_t           b = tt + s * Cfg::TPT;
    return (b / c) * R * c + (b % c) + k * c;
}

// Where element j of the transform that the handle `w` names lives in LDS.  Rows of a tile:
// w is the transform's index in the tile.  FkStrideAddr: w is the LDS index of element 0 and
// the elements are STRIDE apart (the columns of a 2D tile held row by row).
template <typename Cfg>
struct FkRowAddr
{
    static FFT_DEV uint32_t at(uint32_t w, uint32_t j)
    {
        return fk_addr<Cfg>(w, j);
    }
};
template <int STRIDE>
struct FkStrideAddr
{
    static FFT_DEV uint32_t at(uint32_t base, uint32_t j)
    {
        return base + j * (uint32_t)STRIDE;
    }
};

template <typename T, typename Cfg, int P, typename A = FkRowAddr<Cfg>>
FFT_DEV void fk_read(const typename cplx_of<T>::type* lds, uint32_t w, uint32_t tt,
                     typename cplx_of<T>::type* r)
{
    constexpr int R = Cfg::radix(P);
    constexpr int S = Cfg::S(P);
#pragma unroll
    for(int s = 0; s < S; ++s)
        if(fk_live<Cfg, P>(tt, s))
        {
#pragma unroll
            for(int k = 0; k < R; ++k)
                r[s * R + k] = lds[A::at(w, fk_in_pos<Cfg, P>(tt, s, k))];
        }
}

template <typename T, typename Cfg, int P, typename A = FkRowAddr<Cfg>>
FFT_DEV void fk_write(typename cplx_of<T>::type* lds, uint32_t w, uint32_t tt,
                      const typename cplx_of<T>::type* r)
{
    constexpr int R = Cfg::radix(P);
    constexpr int S = Cfg::S(P);
#pragma unroll
    for(int s = 0; s < S; ++s)
        if(fk_live<Cfg, P>(tt, s))
        {
#pragma unroll
            for(int k = 0; k < R; ++k)
                lds[A::at(w, fk_out_pos<Cfg, P>(tt, s, k))] = r[s * R + k];
        }
}

// pass 0 (no twiddles) on register data
template <typename T, typename Cfg>
FFT_DEV void fk_compute0(uint32_t tt, typename cplx_of<T>::type* r)
{
    constexpr int R = Cfg::radix(0);
    constexpr int S = Cfg::S(0);
#pragma unroll
    for(int s = 0; s < S; ++s)
        if(fk_live<Cfg, 0>(tt, s))
            Butterfly<T, R>::run(r + s * R);
}

// The twiddles of pass P (P > 0) as registers (tw_all: the stacked twiddle table of the schedule): fk_twiddles issues the loads, fk_compute_tw uses
// them.  Issued before the LDS exchange that precedes the pass, the loads are in flight while the
// workgroup writes, waits at the barrier and reads (idle slots read the first entry).
template <typename Cfg, int P>
constexpr int fk_tw_count()
{
    return P > 0 && P < Cfg::NP ? Cfg::S(P) * (Cfg::radix(P) - 1) : 1;
}
template <typename T, typename Cfg, int P>
FFT_DEV void fk_twiddles(const void* tw_all, uint32_t tt, typename cplx_of<T>::type* t)
{
    typedef typename cplx_of<T>::type C;
    constexpr int                     R = Cfg::radix(P);
    constexpr int                     S = Cfg::S(P);
    constexpr uint32_t                c = Cfg::cum(P);
    const C* tw = static_cast<const C*>(tw_all) + Cfg::twoff(P);
#pragma unroll
    for(int s = 0; s < S; ++s)
    {
        const uint32_t bl = fk_live<Cfg, P>(tt, s) ? (tt + s * Cfg::TPT) % c : 0u;
#pragma unroll
        for(int k = 1; k < R; ++k)
            t[s * (R - 1) + k - 1] = tw[(k - 1) * c + bl];
    }
}
template <typename T, typename Cfg, int P>
FFT_DEV void fk_compute_tw(const typename cplx_of<T>::type* t, uint32_t tt, typename cplx_of<T>::type* r)
{
    constexpr int R = Cfg::radix(P);
    constexpr int S = Cfg::S(P);
#pragma unroll
    for(int s = 0; s < S; ++s)
    {
        if(!fk_live<Cfg, P>(tt, s))
            continue;
#pragma unroll
        for(int k = 1; k < R; ++k)
            r[s * R + k] = c_mul(r[s * R + k], t[s * (R - 1) + k - 1]);
        Butterfly<T, R>::run(r + s * R);
    }
}

// Workgroup barrier that orders LDS traffic only.  The exchanges between passes communicate
// through LDS alone, so global loads that are in flight (table entries requested ahead of their
// use) need not complete here, as they would have to at a __syncthreads().
__device__ __forceinline__ void fk_lds_barrier()
{
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#endif
}

// all passes on register data; on entry r holds the inputs of pass 0, on exit
// the outputs of the last pass (element (s,k) at fk_out_pos<last>)
template <typename T, typename Cfg, typename A = FkRowAddr<Cfg>>
__device__ __forceinline__ void fk_passes_tw(const void* tw_all, typename cplx_of<T>::type* lds,
                                             uint32_t w, uint32_t tt, bool active,
                                             typename cplx_of<T>::type* r, bool lds_busy)
{
    typedef typename cplx_of<T>::type C;
#define FK_SYNC() fk_lds_barrier()
    if(active)
        fk_compute0<T, Cfg>(tt, r);
    if constexpr(Cfg::NP > 1)
    {
        C t1[fk_tw_count<Cfg, 1>()];
        if(active)
            fk_twiddles<T, Cfg, 1>(tw_all, tt, t1);
        if(lds_busy)
            FK_SYNC();
        if(active)
            fk_write<T, Cfg, 0, A>(lds, w, tt, r);
        FK_SYNC();
        if(active)
        {
            fk_read<T, Cfg, 1, A>(lds, w, tt, r);
            fk_compute_tw<T, Cfg, 1>(t1, tt, r);
        }
    }
    if constexpr(Cfg::NP > 2)
    {
        C t2[fk_tw_count<Cfg, 2>()];
        if(active)
            fk_twiddles<T, Cfg, 2>(tw_all, tt, t2);
        FK_SYNC();
        if(active)
            fk_write<T, Cfg, 1, A>(lds, w, tt, r);
        FK_SYNC();
        if(active)
        {
            fk_read<T, Cfg, 2, A>(lds, w, tt, r);
            fk_compute_tw<T, Cfg, 2>(t2, tt, r);
        }
    }
    if constexpr(Cfg::NP > 3)
    {
        C t3[fk_tw_count<Cfg, 3>()];
        if(active)
            fk_twiddles<T, Cfg, 3>(tw_all, tt, t3);
        FK_SYNC();
        if(active)
            fk_write<T, Cfg, 2, A>(lds, w, tt, r);
        FK_SYNC();
        if(active)
        {
            fk_read<T, Cfg, 3, A>(lds, w, tt, r);
            fk_compute_tw<T, Cfg, 3>(t3, tt, r);
        }
    }
}

template <typename T, typename Cfg>
__device__ __forceinline__ void fk_passes(const fftk_params& p, typename cplx_of<T>::type* lds,
                                          uint32_t w, uint32_t tt, bool active,
                                          typename cplx_of<T>::type* r, bool lds_busy)
{
    fk_passes_tw<T, Cfg>(p.tw, lds, w, tt, active, r, lds_busy);
}

// Global-memory accessors of the lean path.  A side is either an array of interleaved
// (re, im) pairs or two arrays, one of real and one of imaginary parts (planar); offsets count
// complex elements.  at2/put2 take a wave-uniform 64-bit part and a 32-bit lane part.
template <typename T>
struct FkPairsIn
{
    typedef typename cplx_of<T>::type C;
    const C* p;     // element 0 of the tile
    const C* first; // element 0 of the array
    FFT_DEV C at(uint32_t off) const
    {
        return p[off];
    }
    FFT_DEV C at2(uint64_t a, uint32_t b) const
    {
        const C* pk = p + a;
        return pk[b];
    }
    FFT_DEV C at_or_first(bool valid, uint32_t off) const
    {
        const C* pj = valid ? p + off : first;
        return *pj;
    }
};
template <typename T>
struct FkPlanarIn
{
    typedef typename cplx_of<T>::type C;
    const T *re, *im, *first_re, *first_im;
    FFT_DEV C at(uint32_t off) const
    {
        C v;
        v.x = re[off];
        v.y = im[off];
        return v;
    }
    FFT_DEV C at2(uint64_t a, uint32_t b) const
    {
        const T *pr = re + a, *pi = im + a;
        C        v;
        v.x = pr[b];
        v.y = pi[b];
        return v;
    }
    FFT_DEV C at_or_first(bool valid, uint32_t off) const
    {
        const T *pr = valid ? re + off : first_re, *pi = valid ? im + off : first_im;
        C        v;
        v.x = *pr;
        v.y = *pi;
        return v;
    }
};
// real samples (offsets count scalars); the imaginary part reads as zero
template <typename T>
struct FkRealIn
{
    typedef typename cplx_of<T>::type C;
    const T *re, *first_re;
    FFT_DEV C at_or_first(bool valid, uint32_t off) const
    {
        const T* pr = valid ? re + off : first_re;
        C        v;
        v.x = *pr;
        v.y = 0;
        return v;
    }
};
template <typename T>
struct FkPairsOut
{
    typedef typename cplx_of<T>::type C;
    C* p;
    FFT_DEV void put(uint32_t off, C v) const
    {
        p[off] = v;
    }
    FFT_DEV void put2(uint64_t a, uint32_t b, C v) const
    {
        C* pk = p + a;
        pk[b] = v;
    }
};
// The same arrays accessed with the nontemporal hint: data that will not be read again before
// the caches have turned over (the passes of transforms far larger than the last-level cache).
template <typename T>
struct FkPairsInNT
{
    typedef typename cplx_of<T>::type C;
    typedef T                         V __attribute__((ext_vector_type(2)));
    const C*                          p;
    const C*                          first;
    static FFT_DEV C ld(const C* q)
    {
        V v = __builtin_nontemporal_load(reinterpret_cast<const V*>(q));
        C r;
        r.x = v.x;
        r.y = v.y;
        return r;
    }
    FFT_DEV C at(uint32_t off) const
    {
        return ld(p + off);
    }
    FFT_DEV C at2(uint64_t a, uint32_t b) const
    {
        const C* pk = p + a;
        return ld(pk + b);
    }
    FFT_DEV C at_or_first(bool valid, uint32_t off) const
    {
        const C* pj = valid ? p + off : first;
        return ld(pj);
    }
};
template <typename T>
struct FkPairsOutNT
{
    typedef typename cplx_of<T>::type C;
    typedef T                         V __attribute__((ext_vector_type(2)));
    C*                                p;
    static FFT_DEV void st(C* q, C v)
    {
        V w = {v.x, v.y};
        __builtin_nontemporal_store(w, reinterpret_cast<V*>(q));
    }
    FFT_DEV void put(uint32_t off, C v) const
    {
        st(p + off, v);
    }
    FFT_DEV void put2(uint64_t a, uint32_t b, C v) const
    {
        C* pk = p + a;
        st(pk + b, v);
    }
};
template <typename T>
struct FkPlanarOut
{
    typedef typename cplx_of<T>::type C;
    T *re, *im;
    FFT_DEV void put(uint32_t off, C v) const
    {
        re[off] = v.x;
        im[off] = v.y;
    }
    FFT_DEV void put2(uint64_t a, uint32_t b, C v) const
    {
        T *pr = re + a, *pi = im + a;
        pr[b] = v.x;
        pi[b] = v.y;
    }
};

// interleaved pairs of IEEE half values (the arrays of a half-precision plan, which computes in
// single precision): converted on the way in and rounded on the way out
template <typename T>
struct FkHalfIn
{
    typedef typename cplx_of<T>::type C;
    const fft_half2* p;
    const fft_half2* first;
    static FFT_DEV C widen(fft_half2 h)
    {
        C v;
        v.x = (T)h.x;
        v.y = (T)h.y;
        return v;
    }
    FFT_DEV C at(uint32_t off) const
    {
        return widen(p[off]);
    }
    FFT_DEV C at2(uint64_t a, uint32_t b) const
    {
        const fft_half2* pk = p + a;
        return widen(pk[b]);
    }
    FFT_DEV C at_or_first(bool valid, uint32_t off) const
    {
        const fft_half2* pj = valid ? p + off : first;
        return widen(*pj);
    }
};
template <typename T>
struct FkHalfOut
{
    typedef typename cplx_of<T>::type C;
    fft_half2* p;
    static FFT_DEV fft_half2 narrow(C v)
    {
        fft_half2 h;
        h.x = (_Float16)v.x;
        h.y = (_Float16)v.y;
        return h;
    }
    FFT_DEV void put(uint32_t off, C v) const
    {
        p[off] = narrow(v);
    }
    FFT_DEV void put2(uint64_t a, uint32_t b, C v) const
    {
        fft_half2* pk = p + a;
        pk[b]         = narrow(v);
    }
};

// only the real part is written (offsets count scalars)
template <typename T>
struct FkRealOut
{
    typedef typename cplx_of<T>::type C;
    T* re;
    FFT_DEV void put2(uint64_t a, uint32_t b, C v) const
    {
        T* pr = re + a;
        pr[b] = v.x;
    }
};

// element offset of tile entry w of the workgroup (lean path: 32-bit, strides in elements)
template <typename T>
FFT_DEV uint32_t fk_w_in(const fftk_params& p, const TileCtx<T>& c, uint32_t w)
{
    if(!p.w_inner)
        return w * p.w_is_c;
    const uint32_t g = c.tile0 + w, b = g / p.w_inner;
    return (b - c.b0) * p.w2_is_c + (g - b * p.w_inner) * p.w_is_c;
}
template <typename T>
FFT_DEV uint32_t fk_w_out(const fftk_params& p, const TileCtx<T>& c, uint32_t w)
{
    if(!p.w_inner)
        return w * p.w_os_c;
    const uint32_t g = c.tile0 + w, b = g / p.w_inner;
    return (b - c.b0) * p.w2_os_c + (g - b * p.w_inner) * p.w_os_c;
}

// The large twiddles W_L^{j q} of a thread's outputs j = ot + s TPT + k CL of the last pass, in
// factored form: W^{q ot} . W^{q s TPT} . W^{q (k mod 4) CL} . W^{q 4 (k div 4) CL} (the last two
// as one factor for radices up to 4).  A thread with S x R outputs looks up
// 1 + (S-1) + 3 + (ceil(R/4)-1) table values instead of S R of them -- 7 instead of 16 for 64
// points in 4 threads, or for one radix-16 butterfly a thread; 8 instead of 17 for radix 17 --
// and every twiddle is the product of at most four table values, each the product of the two
// entries of the two-level table.  The lookups depend only on the thread's place in the tile,
// so a kernel can issue them before it loads its data (fetch) and form the table values while
// the data is on its way (combine); the dependent round trip to the tables then no longer sits
// between the last butterfly and the stores.
template <typename T, typename Cfg>
struct FkStoreTwiddles
{
    typedef typename cplx_of<T>::type C;
    static constexpr int              LAST   = Cfg::NP - 1;
    static constexpr int              RL     = Cfg::radix(LAST);
    static constexpr int              SL     = Cfg::S(LAST);
    static constexpr int              CL     = Cfg::N / RL;
    static constexpr bool             SPLITK = RL > 4;
    static constexpr int              KL     = SPLITK ? 4 : RL;
    static constexpr int              KH     = SPLITK ? (RL + 3) / 4 : 1;
    static constexpr int              NL     = 1 + (SL - 1) + (KL - 1) + (KH - 1);
    C                                 f[NL], g[NL];
    FFT_DEV void fetch(const fftk_params& p, uint32_t ot, uint32_t oq)
    {
        const C*       tbl  = static_cast<const C*>(p.ltw);
        const uint32_t mask = (1u << p.ltw_shift) - 1u;
        auto           look = [&](int i, uint32_t u) __attribute__((always_inline))
        {
            f[i] = tbl[u & mask];
            g[i] = tbl[(1u << p.ltw_shift) + (u >> p.ltw_shift)];
        };
        look(0, ot * oq);
#pragma unroll
        for(int s = 1; s < SL; ++s)
            look(s, (uint32_t)(s * Cfg::TPT) * oq);
#pragma unroll
        for(int k = 1; k < KL; ++k)
            look(SL - 1 + k, (uint32_t)(k * CL) * oq);
#pragma unroll
        for(int k = 1; k < KH; ++k)
            look(SL + KL - 2 + k, (uint32_t)(4 * k * CL) * oq);
    }
    FFT_DEV void combine()
    {
#pragma unroll
        for(int i = 0; i < NL; ++i)
            f[i] = c_mul(f[i], g[i]);
    }
    // twiddle of output (s, k); s and k are compile-time constants once the callers' loops are unrolled
    FFT_DEV C at(int s, int k) const
    {
        const int kl = SPLITK ? (k & 3) : k, kh = SPLITK ? (k >> 2) : 0;
        C         t  = f[0];
        if(s)
            t = c_mul(t, f[s]);
        if(kl)
            t = c_mul(t, f[SL - 1 + kl]);
        if(kh)
            t = c_mul(t, f[SL + KL - 2 + kh]);
        return t;
    }
};

// Lean path: both sides are complex arrays (interleaved pairs, or planar: in_planar /
// out_planar) whose element offsets inside a
// tile fit 32 bits.  Every address is a wave-uniform 64-bit base plus a 32-bit per-lane
// element offset and there is no per-element branching on the operation kind, so the loads
// of a thread issue back to back.  Covers plain passes, the large twiddle, scaling, the
// Bluestein chirp on either side, convolution mode, the fused real pre/post-processing,
// row-in/column-out passes and (odd lengths) real samples on one side with the half spectrum
// on the other.
// EARLY_TW: the lookups of the large twiddle on the store side are issued before the data loads.
// (The chirp values of the store side stay where they are used: requested early they cost up to
// 64 registers, and the last pass of a 1000003-point single-precision chirp-z transform went
// from 0.115 to 0.149 ms on MI355X with three waves a SIMD instead of four.)
template <typename T, typename Cfg, bool HALF = false, bool EARLY_TW = false>
__device__ __forceinline__ void fast_tile_lean(const fftk_params& p, typename cplx_of<T>::type* lds,
                                               const TileCtx<T>& c, uint32_t tid, uint32_t w,
                                               uint32_t tt, bool active)
{
    typedef typename cplx_of<T>::type C;
    constexpr int                     N    = Cfg::N;
    constexpr int                     LAST = Cfg::NP - 1;
    constexpr int                     RL   = Cfg::radix(LAST);
    constexpr int                     SL   = Cfg::S(LAST);
    constexpr int                     CL   = N / RL; // output (s,k) of the last pass is element tt + s*TPT + k*CL
    constexpr int                     R0   = Cfg::radix(0);
    constexpr int                     S0   = Cfg::S(0);
    constexpr int                     M0   = N / R0; // input (s,k) of pass 0 is element tt + s*TPT + k*M0
    constexpr int                     PAIRS      = (N + 1) / 2; // bins j paired with N-j (j = 0 pairs with N)
    constexpr int                     PAIR_IT    = (PAIRS + Cfg::TPT - 1) / Cfg::TPT;
    constexpr bool                    PAIR_EXACT = PAIRS % Cfg::TPT == 0;
    // transforms whose lanes cover 16 contiguous bytes or less can go through LDS instead
    // (16 bytes of interleaved pairs, or of the scalars of a planar array)
    constexpr bool                    STAGE_OK = Cfg::TPT == 1 || Cfg::TPT * sizeof(C) <= 32;
    constexpr int                     STAGE_IT = (N + Cfg::TPT - 1) / Cfg::TPT;
    constexpr int                     BINS_IT  = (N + 1 + Cfg::TPT - 1) / Cfg::TPT; // N+1 Hermitian bins per row
    // odd lengths also serve as odd-length real transforms (real samples on one side)
    constexpr bool                    ODD_REAL = N % 2 == 1;
    const bool                        ok   = active && (c.tile0 + w < p.tile_cnt);
    const bool                        inv  = p.dir > 0;
    const C*       src = reinterpret_cast<const C*>(static_cast<const T*>(p.in0) + c.ibase);
    C*             dst = reinterpret_cast<C*>(static_cast<T*>(p.out0) + c.obase);
    const uint32_t q   = p.aux_dim == 1 ? (c.tile0 + w) >> p.aux_shift : c.q_block;
    C              r[Cfg::EPT];
    bool           lds_busy = false;
    const FkPairsIn<T>   in_pairs{src, reinterpret_cast<const C*>(static_cast<const T*>(p.in0))};
    const FkPlanarIn<T>  in_planar{static_cast<const T*>(p.in0) + c.ibase, static_cast<const T*>(p.in1) + c.ibase,
                                  static_cast<const T*>(p.in0), static_cast<const T*>(p.in1)};
    const FkPairsOut<T>  out_pairs{dst};
    const FkPairsInNT<T>  in_pairs_nt{src, reinterpret_cast<const C*>(static_cast<const T*>(p.in0))};
    const FkPairsOutNT<T> out_pairs_nt{dst};
    // (HALF: in0 / out0 may point at half values; ibase / obase count scalars of that array)
    const FkHalfIn<T>    in_half{reinterpret_cast<const fft_half2*>(static_cast<const _Float16*>(p.in0) + c.ibase),
                              static_cast<const fft_half2*>(p.in0)};
    const FkHalfOut<T>   out_half{reinterpret_cast<fft_half2*>(static_cast<_Float16*>(p.out0) + c.obase)};
    const FkPlanarOut<T> out_planar{static_cast<T*>(p.out0) + c.obase, static_cast<T*>(p.out1) + c.obase};
// runs body(accessor) with the accessor of the side's array kind
#define FK_WITH_IN(body)            \
    do                              \
    {                               \
        if(HALF && p.in_half)       \
        {                           \
            if constexpr(HALF)      \
                body(in_half);      \
        }                           \
        else if(p.in_planar)        \
            body(in_planar);        \
        else if(p.in_nt)            \
            body(in_pairs_nt);      \
        else                        \
            body(in_pairs);         \
    } while(0)
#define FK_WITH_OUT(body)           \
    do                              \
    {                               \
        if(HALF && p.out_half)      \
        {                           \
            if constexpr(HALF)      \
                body(out_half);     \
        }                           \
        else if(p.out_planar)       \
            body(out_planar);       \
        else if(p.out_nt)           \
            body(out_pairs_nt);     \
        else                        \
            body(out_pairs);        \
    } while(0)

    // The table values of the large twiddle on the store side depend on the thread's place in the
    // tile only and are requested here, before the data (the store section works the place out
    // again below).
    FkStoreTwiddles<T, Cfg> stw;
    if constexpr(EARLY_TW)
    {
        if(p.flags & FFTK_F_TWIDDLE_STORE)
        {
            uint32_t ow0 = w, ot0 = tt;
            if(!p.direct_out)
            {
                if(p.wfast)
                {
                    ot0 = tid % (uint32_t)Cfg::TPT;
                    ow0 = tid / (uint32_t)Cfg::TPT;
                }
                else
                {
                    ow0 = tid & (p.W - 1);
                    ot0 = tid >> p.wshift;
                }
            }
            // (entries beyond the tile read the table at index 0)
            const bool     in_tile = active && (c.tile0 + ow0 < p.tile_cnt);
            const uint32_t oq0     = p.aux_dim == 1 ? (c.tile0 + ow0) >> p.aux_shift : c.q_block;
            stw.fetch(p, in_tile ? ot0 : 0u, in_tile ? oq0 * p.ltw_qmul + p.ltw_qadd : 0u);
        }
    }
    // ---------------------------------------------------------------- load
    if(p.load_op == FFTK_LOAD_C2R_PRE)
    {
        // Hermitian bins -> half-length complex input (library/src/device/kernels/
        // real2complex_device.h:212-254).  A thread takes the pairs (j, N-j), j = tt + TPT*i < (N+1)/2,
        // writes z_j and z_{N-j} to LDS in natural order; pass 0 then reads from LDS.  An even N
        // has the unpaired bin N/2 besides.
        const C*       htw = static_cast<const C*>(p.half_tw);
        const uint32_t wo  = fk_w_in<T>(p, c, w);
        bool           staged = false;
        // the bins of this thread's pairs (ga: bin j, gb: bin N-j, gm: bin N/2) and their twiddles;
        // every load is issued before the first value is used, pairs beyond the row read pair 0
        C              ga[PAIR_IT], gb[PAIR_IT], gt[PAIR_IT], gm;
        gm.x = gm.y = 0;
        if(ok)
        {
#pragma unroll
            for(int i = 0; i < PAIR_IT; ++i)
            {
                const uint32_t j = tt + i * Cfg::TPT;
                gt[i]            = htw[(!PAIR_EXACT && j >= (uint32_t)PAIRS) ? 0u : j];
            }
        }
        if constexpr(STAGE_OK)
        {
            if(p.stage_io)
            {
                // short transforms: consecutive lanes copy consecutive bins of the tile's rows
                // (N+1 each) into LDS, then every thread takes its pairs from there
                staged               = true;
                const uint32_t total = p.W * (uint32_t)(N + 1);
                C              cp[BINS_IT];
                auto           copy_in = [&](auto in) __attribute__((always_inline))
                {
#pragma unroll
                    for(int i = 0; i < BINS_IT; ++i)
                    {
                        const uint32_t e     = tid + i * p.nthreads;
                        const uint32_t w_    = e / (uint32_t)(N + 1);
                        const uint32_t j_    = e - w_ * (uint32_t)(N + 1);
                        const bool     valid = e < total && c.tile0 + w_ < p.tile_cnt;
                        cp[i]                = in.at(valid ? j_ * p.t_is_c + w_ * p.w_is_c : 0u);
                    }
                };
                FK_WITH_IN(copy_in);
                // unconditional stores (a condition would pull each load next to its store and make
                // the thread wait for one load after the other): the LDS allocation of such a pass
                // covers BINS_IT * nthreads elements
#pragma unroll
                for(int i = 0; i < BINS_IT; ++i)
                    lds[tid + i * p.nthreads] = cp[i];
                fk_lds_barrier();
                if(ok)
                {
                    const uint32_t row = w * (uint32_t)(N + 1);
#pragma unroll
                    for(int i = 0; i < PAIR_IT; ++i)
                    {
                        const uint32_t j = tt + i * Cfg::TPT;
                        if(!PAIR_EXACT && j >= (uint32_t)PAIRS)
                            continue;
                        ga[i] = lds[row + j];
                        gb[i] = lds[row + (uint32_t)N - j];
                    }
                    if(N % 2 == 0 && tt == 0)
                        gm = lds[row + N / 2];
                }
                fk_lds_barrier();
            }
        }
        auto fetch_pairs = [&](auto in) __attribute__((always_inline))
        {
#pragma unroll
            for(int i = 0; i < PAIR_IT; ++i)
            {
                const uint32_t j  = tt + i * Cfg::TPT;
                const uint32_t js = (!PAIR_EXACT && j >= (uint32_t)PAIRS) ? 0u : j;
                ga[i]             = in.at(js * p.t_is_c + wo);
                gb[i]             = in.at(((uint32_t)N - js) * p.t_is_c + wo);
            }
            if(N % 2 == 0 && tt == 0)
                gm = in.at((N / 2) * p.t_is_c + wo);
        };
        if(ok && !staged)
            FK_WITH_IN(fetch_pairs);
        if(ok)
        {
#pragma unroll
            for(int i = 0; i < PAIR_IT; ++i)
            {
                const uint32_t j  = tt + i * Cfg::TPT;
                const uint32_t jq = N - j;
                if(!PAIR_EXACT && j >= (uint32_t)PAIRS)
                    continue;
                const C        a = ga[i], bq = gb[i];
                C              zj, zq;
                if(j == 0)
                {
                    zj.x = a.x + bq.x;
                    zj.y = a.x - bq.x;
                }
                else
                {
                    C t  = gt[i];
                    C u  = c_add(a, bq);
                    C v  = c_sub(a, bq);
                    zj.x = u.x + v.x * t.y - u.y * t.x;
                    zj.y = v.y + u.y * t.y + v.x * t.x;
                    zq.x = u.x - v.x * t.y + u.y * t.x;
                    zq.y = -v.y + u.y * t.y + v.x * t.x;
                    lds[fk_addr<Cfg>(w, jq)] = c_swap(zq);
                }
                lds[fk_addr<Cfg>(w, j)] = c_swap(zj);
            }
            if(N % 2 == 0 && tt == 0)
            {
                C z;
                z.x                         = (T)2 * gm.x;
                z.y                         = (T)-2 * gm.y;
                lds[fk_addr<Cfg>(w, N / 2)] = c_swap(z);
            }
        }
        fk_lds_barrier();
        if(active)
            fk_read<T, Cfg, 0>(lds, w, tt, r);
        lds_busy = true;
    }
    else if(ODD_REAL && p.load_op == FFTK_LOAD_REAL && !(p.flags & FFTK_F_CHIRP_LOAD))
    {
        // odd-length real forward: real samples (strides in scalars), imaginary parts zero
        const T*       srcr = static_cast<const T*>(p.in0) + c.ibase;
        const uint32_t li   = tt * p.t_is_c + fk_w_in<T>(p, c, w);
        if(ok)
        {
#pragma unroll
            for(int s = 0; s < S0; ++s)
#pragma unroll
                for(int k = 0; k < R0; ++k)
                {
                    const T* pk = srcr + (uint64_t)(s * Cfg::TPT + k * M0) * p.t_is_c;
                    if(fk_live<Cfg, 0>(tt, s))
                    {
                        C v;
                        v.x           = pk[li];
                        v.y           = 0;
                        r[s * R0 + k] = inv ? c_swap(v) : v;
                    }
                }
        }
    }
    else if(ODD_REAL && p.load_op == FFTK_LOAD_HERM_EXPAND && !(p.flags & FFTK_F_CHIRP_LOAD))
    {
        // odd-length real inverse: bins 0..N/2 are stored, bin j > N/2 is the conjugate of bin
        // N-j; the imaginary part of bin 0 is ignored
        const uint32_t wo = fk_w_in<T>(p, c, w);
        auto expand = [&](auto in) __attribute__((always_inline))
        {
#pragma unroll
            for(int s = 0; s < S0; ++s)
#pragma unroll
                for(int k = 0; k < R0; ++k)
                {
                    const uint32_t j  = tt + s * Cfg::TPT + k * M0;
                    const uint32_t jm = j <= (uint32_t)(N / 2) ? j : (uint32_t)N - j;
                    if(fk_live<Cfg, 0>(tt, s))
                    {
                        C v = in.at(jm * p.t_is_c + wo);
                        if(jm != j)
                            v.y = -v.y;
                        if(j == 0)
                            v.y = 0;
                        r[s * R0 + k] = inv ? c_swap(v) : v;
                    }
                }
        };
        if(ok)
            FK_WITH_IN(expand);
    }
    else if(STAGE_OK && p.stage_io)
    {
        // consecutive lanes copy consecutive elements of the tile into LDS
        const uint32_t total = p.W * N;
        // every load is issued before the first value is used
        C    cp[STAGE_IT];
        auto copy_in = [&](auto in) __attribute__((always_inline))
        {
#pragma unroll
            for(int i = 0; i < STAGE_IT; ++i)
            {
                const uint32_t e     = tid + i * p.nthreads;
                const uint32_t w_    = e / (uint32_t)N;
                const uint32_t j_    = e - w_ * (uint32_t)N;
                const bool     valid = e < total && c.tile0 + w_ < p.tile_cnt;
                cp[i]                = in.at(valid ? j_ * p.t_is_c + w_ * p.w_is_c : 0u);
            }
        };
        FK_WITH_IN(copy_in);
        // unconditional stores, as above: the LDS allocation covers the rows up to
        // (STAGE_IT * nthreads - 1) / N
#pragma unroll
        for(int i = 0; i < STAGE_IT; ++i)
        {
            const uint32_t e  = tid + i * p.nthreads;
            const uint32_t w_ = e / (uint32_t)N;
            const uint32_t j_ = e - w_ * (uint32_t)N;
            lds[fk_addr<Cfg>(w_, j_)] = inv ? c_swap(cp[i]) : cp[i];
        }
        fk_lds_barrier();
        if(active)
            fk_read<T, Cfg, 0>(lds, w, tt, r);
        lds_busy = true;
    }
    else
    {
        const uint32_t li = tt * p.t_is_c + fk_w_in<T>(p, c, w);
        if(ok)
        {
            if(p.flags & FFTK_F_CHIRP_LOAD)
            {
                // samples beyond the signal read as zero; their loads are redirected to the
                // first element of the array instead of being skipped, so that all loads stay in
                // flight (not to the first sample of this tile: the tile itself lies beyond the
                // array when the table-indexed axis is longer than the signal)
                const C*   chirp = static_cast<const C*>(p.chirp);
                const bool cj    = (p.flags & FFTK_F_CHIRP_CONJ) != 0;
                C          ch[Cfg::EPT];
                const bool herm  = p.load_op == FFTK_LOAD_HERM_EXPAND;
                const uint32_t win = fk_w_in<T>(p, c, w);
                auto       fetch = [&](auto in) __attribute__((always_inline))
                {
#pragma unroll
                    for(int s = 0; s < S0; ++s)
#pragma unroll
                        for(int k = 0; k < R0; ++k)
                        {
                            const uint32_t j     = tt + s * Cfg::TPT + k * M0;
                            const uint32_t idx   = j * p.chirp_js + q * p.chirp_qs;
                            const bool     valid = idx < p.blu_n && fk_live<Cfg, 0>(tt, s);
                            // Hermitian input of an odd-length real inverse transform (chirp index =
                            // sample index there): bins above n_in/2 are the conjugate mirror
                            const uint32_t jm = (herm && j > p.n_in / 2) ? p.n_in - j : j;
                            // (a slot that is padding for every lane of the wave loads nothing: half
                            // of a power-of-two convolution length is padding)
#if defined(__HIP_DEVICE_COMPILE__)
                            const bool any_valid = __builtin_amdgcn_ballot_w64(valid) != 0;
#else
                            const bool any_valid = valid;
#endif
                            C v, cv;
                            v.x = v.y = cv.x = cv.y = 0;
                            if(any_valid)
                            {
                                v  = in.at_or_first(valid, jm * p.t_is_c + win);
                                cv = chirp[valid ? idx : 0u];
                            }
                            if(herm)
                            {
                                if(jm != j)
                                    v.y = -v.y;
                                if(j == 0 || 2 * j == p.n_in)
                                    v.y = 0;
                            }
                            r[s * R0 + k]  = v;
                            ch[s * R0 + k] = cv;
                        }
                };
                if(p.load_op == FFTK_LOAD_REAL)
                    fetch(FkRealIn<T>{static_cast<const T*>(p.in0) + c.ibase, static_cast<const T*>(p.in0)});
                else
                    FK_WITH_IN(fetch);
#pragma unroll
                for(int s = 0; s < S0; ++s)
#pragma unroll
                    for(int k = 0; k < R0; ++k)
                    {
                        const uint32_t j   = tt + s * Cfg::TPT + k * M0;
                        const uint32_t idx = j * p.chirp_js + q * p.chirp_qs;
                        C              x   = r[s * R0 + k];
                        C v = cj ? c_mul(x, ch[s * R0 + k]) : c_mulc(x, ch[s * R0 + k]);
                        if(idx >= p.blu_n)
                        {
                            v.x = 0;
                            v.y = 0;
                        }
                        r[s * R0 + k] = v;
                    }
            }
            else
            {
                auto fetch = [&](auto in) __attribute__((always_inline))
                {
#pragma unroll
                    for(int s = 0; s < S0; ++s)
#pragma unroll
                        for(int k = 0; k < R0; ++k)
                            if(fk_live<Cfg, 0>(tt, s))
                                r[s * R0 + k] = in.at2((uint64_t)(s * Cfg::TPT + k * M0) * p.t_is_c, li);
                };
                FK_WITH_IN(fetch);
            }
            if(inv)
            {
#pragma unroll
                for(int i = 0; i < Cfg::EPT; ++i)
                    r[i] = c_swap(r[i]);
            }
        }
    }

    if constexpr(EARLY_TW)
    {
        if(p.flags & FFTK_F_TWIDDLE_STORE)
            stw.combine();
    }
    // ---------------------------------------------------------------- transform(s)
    fk_passes<T, Cfg>(p, lds, w, tt, active, r, lds_busy);
    bool out_inv = inv;
    if(p.flags & FFTK_F_CONV)
    {
        // r holds the forward spectrum: multiply by the stored spectrum, exchange re/im and
        // run the passes again, which makes the second transform an inverse one
        const C* cb = static_cast<const C*>(p.convb) + (uint64_t)q * p.convb_qs;
        if constexpr(RL == R0)
        {
            // equal first and last radix: the last pass leaves a thread exactly the elements
            // its first pass takes (tt + s TPT + k N/R), so the spectrum stays in registers
            if(active)
            {
                // the loads of the stored spectrum are issued together (rows beyond the tile and
                // idle slots read its first element)
                C sp[SL * RL];
#pragma unroll
                for(int s = 0; s < SL; ++s)
#pragma unroll
                    for(int k = 0; k < RL; ++k)
                    {
                        const uint32_t j = tt + s * Cfg::TPT + k * CL;
                        sp[s * RL + k]   = cb[(ok && fk_live<Cfg, LAST>(tt, s)) ? j : 0u];
                    }
#pragma unroll
                for(int s = 0; s < SL; ++s)
#pragma unroll
                    for(int k = 0; k < RL; ++k)
                    {
                        if(!fk_live<Cfg, LAST>(tt, s))
                            continue;
                        r[s * RL + k] = c_swap(c_mul(r[s * RL + k], sp[s * RL + k]));
                    }
            }
            fk_passes<T, Cfg>(p, lds, w, tt, active, r, Cfg::NP > 1 || lds_busy);
        }
        else
        {
            if(Cfg::NP > 1 || lds_busy)
                fk_lds_barrier();
            if(active)
            {
                C sp[SL * RL];
#pragma unroll
                for(int s = 0; s < SL; ++s)
#pragma unroll
                    for(int k = 0; k < RL; ++k)
                    {
                        const uint32_t j = tt + s * Cfg::TPT + k * CL;
                        sp[s * RL + k]   = cb[(ok && fk_live<Cfg, LAST>(tt, s)) ? j : 0u];
                    }
#pragma unroll
                for(int s = 0; s < SL; ++s)
#pragma unroll
                    for(int k = 0; k < RL; ++k)
                    {
                        const uint32_t j = tt + s * Cfg::TPT + k * CL;
                        if(!fk_live<Cfg, LAST>(tt, s))
                            continue;
                        lds[fk_addr<Cfg>(w, j)] = c_swap(c_mul(r[s * RL + k], sp[s * RL + k]));
                    }
            }
            fk_lds_barrier();
            if(active)
                fk_read<T, Cfg, 0>(lds, w, tt, r);
            fk_passes<T, Cfg>(p, lds, w, tt, active, r, true);
        }
        lds_busy = lds_busy || Cfg::NP > 1 || RL != R0;
        out_inv  = true;
    }

    // ---------------------------------------------------------------- store
    if(p.store_op == FFTK_STORE_R2C_POST)
    {
        // half-length spectrum -> N+1 Hermitian bins (real2complex_device.h:25-103): natural
        // order through LDS, then a thread produces the pairs (j, N-j)
        if(Cfg::NP > 1 || lds_busy)
            fk_lds_barrier();
        if(active)
            fk_write<T, Cfg, LAST>(lds, w, tt, r);
        fk_lds_barrier();
        if constexpr(STAGE_OK)
        {
            if(p.stage_io)
            {
                // short transforms: the bins go back to LDS as the image of the tile's output
                // rows (N+1 bins each), which consecutive lanes then copy out
                const C* htw = static_cast<const C*>(p.half_tw);
                const T  sc  = (p.flags & FFTK_F_SCALE) ? (T)p.scale : (T)1;
                C        zp[PAIR_IT], zq[PAIR_IT], zm;
                zm.x = zm.y = 0;
                if(ok)
                {
#pragma unroll
                    for(int i = 0; i < PAIR_IT; ++i)
                    {
                        const uint32_t j = tt + i * Cfg::TPT;
                        if(!PAIR_EXACT && j >= (uint32_t)PAIRS)
                            continue;
                        zp[i] = lds[fk_addr<Cfg>(w, j)];
                        zq[i] = lds[fk_addr<Cfg>(w, j == 0 ? 0u : (uint32_t)N - j)];
                    }
                    if(N % 2 == 0 && tt == 0)
                        zm = lds[fk_addr<Cfg>(w, N / 2)];
                }
                fk_lds_barrier();
                if(ok)
                {
                    const uint32_t row = w * (uint32_t)(N + 1);
#pragma unroll
                    for(int i = 0; i < PAIR_IT; ++i)
                    {
                        const uint32_t j = tt + i * Cfg::TPT;
                        if(!PAIR_EXACT && j >= (uint32_t)PAIRS)
                            continue;
                        C o0, o1;
                        if(j == 0)
                        {
                            o0.x = zp[i].x + zp[i].y;
                            o0.y = 0;
                            o1.x = zp[i].x - zp[i].y;
                            o1.y = 0;
                        }
                        else
                        {
                            C t = htw[j];
                            C u, v;
                            u.x  = (T)0.5 * (zp[i].x + zq[i].x);
                            u.y  = (T)0.5 * (zp[i].y + zq[i].y);
                            v.x  = (T)0.5 * (zp[i].x - zq[i].x);
                            v.y  = (T)0.5 * (zp[i].y - zq[i].y);
                            o0.x = u.x + v.x * t.y + u.y * t.x;
                            o0.y = v.y + u.y * t.y - v.x * t.x;
                            o1.x = u.x - v.x * t.y - u.y * t.x;
                            o1.y = -v.y + u.y * t.y - v.x * t.x;
                        }
                        o0.x *= sc;
                        o0.y *= sc;
                        o1.x *= sc;
                        o1.y *= sc;
                        lds[row + j]               = o0;
                        lds[row + (uint32_t)N - j] = o1;
                    }
                    if(N % 2 == 0 && tt == 0)
                    {
                        C o;
                        o.x              = zm.x * sc;
                        o.y              = -zm.y * sc;
                        lds[row + N / 2] = o;
                    }
                }
                fk_lds_barrier();
                const uint32_t total = p.W * (uint32_t)(N + 1);
                auto copy_out = [&](auto out) __attribute__((always_inline))
                {
#pragma unroll
                    for(int i = 0; i < BINS_IT; ++i)
                    {
                        const uint32_t e  = tid + i * p.nthreads;
                        const uint32_t w_ = e / (uint32_t)(N + 1);
                        const uint32_t j_ = e - w_ * (uint32_t)(N + 1);
                        if(e < total && c.tile0 + w_ < p.tile_cnt)
                            out.put(j_ * p.t_os_c + w_ * p.w_os_c, lds[e]);
                    }
                };
                FK_WITH_OUT(copy_out);
                return;
            }
        }
        auto post_pairs = [&](auto out) __attribute__((always_inline))
        {
            const C*       htw = static_cast<const C*>(p.half_tw);
            const uint32_t wo  = fk_w_out<T>(p, c, w);
            const T        sc  = (p.flags & FFTK_F_SCALE) ? (T)p.scale : (T)1;
            // the twiddle loads of all pairs are issued before the first store (a store could
            // alias a later load and would hold it back)
            C gt[PAIR_IT];
#pragma unroll
            for(int i = 0; i < PAIR_IT; ++i)
            {
                const uint32_t j = tt + i * Cfg::TPT;
                gt[i]            = htw[(!PAIR_EXACT && j >= (uint32_t)PAIRS) ? 0u : j];
            }
#pragma unroll
            for(int i = 0; i < PAIR_IT; ++i)
            {
                const uint32_t j  = tt + i * Cfg::TPT;
                const uint32_t jq = N - j;
                if(!PAIR_EXACT && j >= (uint32_t)PAIRS)
                    continue;
                C              zp = lds[fk_addr<Cfg>(w, j)];
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
                    C zq = lds[fk_addr<Cfg>(w, jq)];
                    C t  = gt[i];
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
                o0.x *= sc;
                o0.y *= sc;
                o1.x *= sc;
                o1.y *= sc;
                out.put(j * p.t_os_c + wo, o0);
                out.put(jq * p.t_os_c + wo, o1);
            }
            if(N % 2 == 0 && tt == 0)
            {
                C z = lds[fk_addr<Cfg>(w, N / 2)];
                C o;
                o.x = z.x * sc;
                o.y = -z.y * sc;
                out.put((N / 2) * p.t_os_c + wo, o);
            }
        };
        if(ok)
            FK_WITH_OUT(post_pairs);
        return;
    }

    if(STAGE_OK && p.stage_io)
    {
        if(Cfg::NP > 1 || lds_busy)
            fk_lds_barrier();
        if(active)
            fk_write<T, Cfg, LAST>(lds, w, tt, r);
        fk_lds_barrier();
        const uint32_t total = p.W * N;
        const T        sc    = (p.flags & FFTK_F_SCALE) ? (T)p.scale : (T)1;
#pragma unroll
        for(int i = 0; i < STAGE_IT; ++i)
        {
            const uint32_t e     = tid + i * p.nthreads;
            const uint32_t w_    = e / (uint32_t)N;
            const uint32_t j_    = e - w_ * (uint32_t)N;
            const bool     valid = e < total && c.tile0 + w_ < p.tile_cnt;
            if(valid)
            {
                C v = lds[fk_addr<Cfg>(w_, j_)];
                if(out_inv)
                    v = c_swap(v);
                v.x *= sc;
                v.y *= sc;
                auto put = [&](auto out) __attribute__((always_inline)) { out.put(j_ * p.t_os_c + w_ * p.w_os_c, v); };
                FK_WITH_OUT(put);
            }
        }
        return;
    }

    uint32_t ow = w, ot = tt;
    bool     ook = ok;
    if(!p.direct_out)
    {
        // the store runs along the other axis than the load did: through LDS in natural
        // order, then re-read with the lanes running along the tile dimension (or along the
        // transform) so that the global stores coalesce
        if(Cfg::NP > 1 || lds_busy)
            fk_lds_barrier();
        if(active)
            fk_write<T, Cfg, LAST>(lds, w, tt, r);
        fk_lds_barrier();
        if(p.wfast)
        {
            ot = tid % (uint32_t)Cfg::TPT;
            ow = tid / (uint32_t)Cfg::TPT;
        }
        else
        {
            ow = tid & (p.W - 1);
            ot = tid >> p.wshift;
        }
        ook = active && (c.tile0 + ow < p.tile_cnt);
        if(active)
        {
#pragma unroll
            for(int s = 0; s < SL; ++s)
#pragma unroll
                for(int k = 0; k < RL; ++k)
                    if(fk_live<Cfg, LAST>(ot, s))
                        r[s * RL + k] = lds[fk_addr<Cfg>(ow, ot + s * Cfg::TPT + k * CL)];
        }
    }
    const uint32_t oq = p.aux_dim == 1 ? (c.tile0 + ow) >> p.aux_shift : c.q_block;
    const uint32_t lo = ot * p.t_os_c + fk_w_out<T>(p, c, ow);
    if(ook)
    {
        if(out_inv)
        {
#pragma unroll
            for(int i = 0; i < Cfg::EPT; ++i)
                r[i] = c_swap(r[i]);
        }
        if(p.flags & FFTK_F_TWIDDLE_STORE)
        {
            if constexpr(!EARLY_TW)
            {
                stw.fetch(p, ot, oq * p.ltw_qmul + p.ltw_qadd);
                stw.combine();
            }
#pragma unroll
            for(int s = 0; s < SL; ++s)
#pragma unroll
                for(int k = 0; k < RL; ++k)
                {
                    const C tv    = stw.at(s, k);
                    r[s * RL + k] = out_inv ? c_mulc(r[s * RL + k], tv) : c_mul(r[s * RL + k], tv);
                }
        }
        if(p.flags & FFTK_F_SCALE)
        {
#pragma unroll
            for(int i = 0; i < Cfg::EPT; ++i)
            {
                r[i].x *= (T)p.scale;
                r[i].y *= (T)p.scale;
            }
        }
        if(p.flags & FFTK_F_CHIRP_STORE)
        {
            const C*   chirp = static_cast<const C*>(p.chirp);
            const bool cj    = (p.flags & FFTK_F_CHIRP_CONJ) != 0;
            C          ch[Cfg::EPT];
#pragma unroll
            for(int s = 0; s < SL; ++s)
#pragma unroll
                for(int k = 0; k < RL; ++k)
                {
                    const uint32_t j    = ot + s * Cfg::TPT + k * CL;
                    const uint32_t idx  = j * p.chirp_js + oq * p.chirp_qs;
                    const bool     keep = idx < p.blu_n && j < p.n_out && fk_live<Cfg, LAST>(ot, s);
#if defined(__HIP_DEVICE_COMPILE__)
                    const bool any_kept = __builtin_amdgcn_ballot_w64(keep) != 0;
#else
                    const bool any_kept = keep;
#endif
                    C cv;
                    cv.x = cv.y = 0;
                    if(any_kept)
                        cv = chirp[keep ? idx : 0u];
                    ch[s * RL + k] = cv;
                }
            auto emit = [&](auto out) __attribute__((always_inline))
            {
#pragma unroll
                for(int s = 0; s < SL; ++s)
#pragma unroll
                    for(int k = 0; k < RL; ++k)
                    {
                        const uint32_t j   = ot + s * Cfg::TPT + k * CL;
                        const uint32_t idx = j * p.chirp_js + oq * p.chirp_qs;
                        C v = cj ? c_mul(r[s * RL + k], ch[s * RL + k]) : c_mulc(r[s * RL + k], ch[s * RL + k]);
                        if(idx < p.blu_n && j < p.n_out && fk_live<Cfg, LAST>(ot, s))
                            out.put2((uint64_t)(s * Cfg::TPT + k * CL) * p.t_os_c, lo, v);
                    }
            };
            if(p.store_op == FFTK_STORE_REAL)
                emit(FkRealOut<T>{static_cast<T*>(p.out0) + c.obase});
            else
                FK_WITH_OUT(emit);
        }
        else if(ODD_REAL && p.store_op == FFTK_STORE_REAL)
        {
            // real parts only (strides in scalars)
            T* dstr = static_cast<T*>(p.out0) + c.obase;
#pragma unroll
            for(int s = 0; s < SL; ++s)
#pragma unroll
                for(int k = 0; k < RL; ++k)
                {
                    T* pk = dstr + (uint64_t)(s * Cfg::TPT + k * CL) * p.t_os_c;
                    if(fk_live<Cfg, LAST>(ot, s))
                        pk[lo] = r[s * RL + k].x;
                }
        }
        else
        {
            auto emit = [&](auto out) __attribute__((always_inline))
            {
#pragma unroll
                for(int s = 0; s < SL; ++s)
#pragma unroll
                    for(int k = 0; k < RL; ++k)
                    {
                        // an odd-length real forward transform keeps the first n_out bins
                        if(fk_live<Cfg, LAST>(ot, s) && (!ODD_REAL || ot + s * Cfg::TPT + k * CL < p.n_out))
                            out.put2((uint64_t)(s * Cfg::TPT + k * CL) * p.t_os_c, lo, r[s * RL + k]);
                    }
            };
            FK_WITH_OUT(emit);
        }
    }
#undef FK_WITH_IN
#undef FK_WITH_OUT
}

template <typename T, typename Cfg, bool VEC, bool LEAN, bool HALF = false, bool EARLY_TW = false>
__device__ __forceinline__ void fast_tile_body(const fftk_params& p, typename cplx_of<T>::type* lds)
{
    typedef typename cplx_of<T>::type C;
    constexpr int                     LAST = Cfg::NP - 1;
    constexpr int                     RL   = Cfg::radix(LAST);
    constexpr int                     SL   = Cfg::S(LAST);
    constexpr int                     R0   = Cfg::radix(0);
    constexpr int                     S0   = Cfg::S(0);
    const uint32_t                    tid  = threadIdx.x;
    TileCtx<T>                        c;
    tile_decode<T>(p, blockIdx.x, c);
    uint32_t w, tt;
    bool     active = tid < (uint32_t)Cfg::TPT * p.W;
    if(p.wfast)
    {
        w  = tid & (p.W - 1);
        tt = tid >> p.wshift;
    }
    else
    {
        tt = tid % (uint32_t)Cfg::TPT;
        w  = tid / (uint32_t)Cfg::TPT;
    }
    if constexpr(LEAN)
    {
        fast_tile_lean<T, Cfg, HALF, EARLY_TW>(p, lds, c, tid, w, tt, active);
        return;
    }
    C    r[Cfg::EPT];
    bool lds_busy;
    if(p.direct_in)
    {
        if(active)
        {
#pragma unroll
            for(int s = 0; s < S0; ++s)
#pragma unroll
                for(int k = 0; k < R0; ++k)
                    if(fk_live<Cfg, 0>(tt, s))
                        r[s * R0 + k] = fetch_elem<T, VEC>(p, c, w, fk_in_pos<Cfg, 0>(tt, s, k));
        }
        lds_busy = false;
    }
    else
    {
        tile_load<T, VEC>(p, c, lds, tid);
        __syncthreads();
        if(active)
            fk_read<T, Cfg, 0>(lds, w, tt, r);
        lds_busy = true;
    }
    fk_passes<T, Cfg>(p, lds, w, tt, active, r, lds_busy);
    if(p.flags & FFTK_F_CONV)
    {
        // r holds the forward spectrum: multiply by the stored spectrum, exchange re/im
        // and run the passes again, which makes the second transform an inverse one
        uint32_t q = p.aux_dim == 1 ? (c.tile0 + w) >> p.aux_shift : c.q_block;
        if(Cfg::NP > 1)
            __syncthreads();
        if(active)
        {
            const bool valid = c.tile0 + w < p.tile_cnt;
#pragma unroll
            for(int s = 0; s < SL; ++s)
#pragma unroll
                for(int k = 0; k < RL; ++k)
                {
                    uint32_t j = fk_out_pos<Cfg, LAST>(tt, s, k);
                    if(!fk_live<Cfg, LAST>(tt, s))
                        continue;
                    C v = r[s * RL + k];
                    if(valid)
                        v = c_mul(v, static_cast<const C*>(p.convb)[j + q * p.convb_qs]);
                    lds[fk_addr<Cfg>(w, j)] = c_swap(v);
                }
        }
        __syncthreads();
        if(active)
            fk_read<T, Cfg, 0>(lds, w, tt, r);
        fk_passes<T, Cfg>(p, lds, w, tt, active, r, true);
    }
    if(p.direct_out)
    {
        if(active)
        {
#pragma unroll
            for(int s = 0; s < SL; ++s)
#pragma unroll
                for(int k = 0; k < RL; ++k)
                    if(fk_live<Cfg, LAST>(tt, s))
                        emit_elem<T, VEC>(p, c, w, fk_out_pos<Cfg, LAST>(tt, s, k), r[s * RL + k]);
        }
    }
    else
    {
        if(Cfg::NP > 1 || !p.direct_in || (p.flags & FFTK_F_CONV))
            __syncthreads();
        if(active)
            fk_write<T, Cfg, LAST>(lds, w, tt, r);
        __syncthreads();
        tile_store<T, VEC>(p, c, lds, tid);
    }
}
#undef FK_SYNC

#endif
