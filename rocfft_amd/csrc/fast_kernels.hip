// fast_kernels.hip -- instantiations of the compile-time-schedule tile kernel
// (fast_core.h) for the lengths listed in fast_schedules.h, and their registry.
//
// The file is compiled FAST_SLICES times with -DFAST_SLICE=0..FAST_SLICES-1; every
// translation unit instantiates the kernels of its slice of the list, and slice 0 also
// holds the lookup over all slices.
#include "fast_core.h"
#include "lds_limit.h"
#include "fast_registry.h"
#include "gpu_rt.h"
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <vector>

#ifndef FAST_SLICE
#error "compile with -DFAST_SLICE=<n>"
#endif

namespace
{

// MODE 0: scalar accesses, every fused operation; 1: vector accesses, every fused operation;
// 2: the lean path (vector accesses, complex arrays on both sides, every fused operation);
// 3: the lean path for plain passes only (interleaved complex in and out, nothing fused but a
// scale factor); 4: interleaved arrays, a scale factor, the large twiddle on the store side, the
// fused real pre/post-processing, the tile copy of short transforms, and (single precision)
// arrays of IEEE half pairs on the load or the store side: the first and last pass of a
// half-precision plan, which computes in single precision; 5 (odd lengths): real samples on one
// side and the half spectrum on the other, nothing else fused but a scale factor; 7, 9 and 8: the
// first, middle and last pass of a chirp-z transform in three kernels (powers of two only).  The
// variants 3, 4, 5, 7, 8, 9 are
// the lean kernel compiled under assumptions on its arguments (fast_assume_plain): the compiler
// drops every other path, which leaves a fifth to a third of the code and 10-50 registers fewer.
// Workgroups have up to 512 threads (row passes use up to 256, strided passes more to keep
// their tile rows wide); no kernel here needs more than the 256 registers that leaves a thread.
// The longest lengths need up to 1024 threads for one transform (128 registers a thread).
template <typename Cfg>
constexpr int fast_block_limit()
{
    return Cfg::TPT > 512 ? 1024 : 512;
}

// what fftrt_launch_fast_tile has checked on the host before it picks variant 3 or 4
template <typename Cfg, int MODE>
__device__ __forceinline__ void fast_assume_plain(const fftk_params& p)
{
    if constexpr(MODE == 4)
    {
        __builtin_assume(p.load_op == FFTK_LOAD_COMPLEX || p.load_op == FFTK_LOAD_C2R_PRE);
        __builtin_assume(p.store_op == FFTK_STORE_COMPLEX || p.store_op == FFTK_STORE_R2C_POST);
        __builtin_assume((p.flags & ~(uint32_t)(FFTK_F_SCALE | FFTK_F_TWIDDLE_STORE)) == 0);
        __builtin_assume(p.in_planar == 0);
        __builtin_assume(p.out_planar == 0);
        __builtin_assume(p.w_inner == 0);
    }
    else if constexpr(MODE == 5)
    {
        // odd-length real transforms: real samples -> half spectrum, or half spectrum -> real samples
        __builtin_assume(p.load_op == FFTK_LOAD_REAL || p.load_op == FFTK_LOAD_HERM_EXPAND);
        __builtin_assume(p.store_op == FFTK_STORE_COMPLEX || p.store_op == FFTK_STORE_REAL);
        __builtin_assume((p.flags & ~(uint32_t)FFTK_F_SCALE) == 0);
        __builtin_assume(p.in_planar == 0);
        __builtin_assume(p.out_planar == 0);
        __builtin_assume(p.stage_io == 0);
        __builtin_assume(p.w_inner == 0);
        __builtin_assume(p.aux_dim == 0);
        __builtin_assume(p.oc0_first == 0);
        __builtin_assume(p.in_nt == 0);
        __builtin_assume(p.out_nt == 0);
    }
    else if constexpr(MODE == 7)
    {
        // first pass of a chirp-z transform in three kernels: chirp and zero padding on the load
        // side, the large twiddle on the store side, interleaved arrays
        __builtin_assume(p.load_op == FFTK_LOAD_COMPLEX);
        __builtin_assume(p.store_op == FFTK_STORE_COMPLEX);
        __builtin_assume((p.flags & ~(uint32_t)(FFTK_F_CHIRP_LOAD | FFTK_F_TWIDDLE_STORE | FFTK_F_CHIRP_CONJ)) == 0);
        __builtin_assume((p.flags & FFTK_F_CHIRP_LOAD) != 0);
        __builtin_assume(p.in_planar == 0);
        __builtin_assume(p.out_planar == 0);
        __builtin_assume(p.stage_io == 0);
        __builtin_assume(p.w_inner == 0);
        __builtin_assume(p.in_nt == 0);
        __builtin_assume(p.out_nt == 0);
    }
    else if constexpr(MODE == 8)
    {
        // last pass of such a transform: chirp and scale factor on the store side
        __builtin_assume(p.load_op == FFTK_LOAD_COMPLEX);
        __builtin_assume(p.store_op == FFTK_STORE_COMPLEX);
        __builtin_assume((p.flags & ~(uint32_t)(FFTK_F_CHIRP_STORE | FFTK_F_SCALE | FFTK_F_CHIRP_CONJ)) == 0);
        __builtin_assume((p.flags & FFTK_F_CHIRP_STORE) != 0);
        __builtin_assume(p.in_planar == 0);
        __builtin_assume(p.out_planar == 0);
        __builtin_assume(p.stage_io == 0);
        __builtin_assume(p.w_inner == 0);
        __builtin_assume(p.n_in == (uint32_t)Cfg::N);
        __builtin_assume(p.in_nt == 0);
        __builtin_assume(p.out_nt == 0);
    }
    else if constexpr(MODE == 9)
    {
        // middle pass of such a transform: forward transform, product with the chirp spectrum,
        // inverse transform, the large twiddle on the store side
        __builtin_assume(p.load_op == FFTK_LOAD_COMPLEX);
        __builtin_assume(p.store_op == FFTK_STORE_COMPLEX);
        __builtin_assume((p.flags & ~(uint32_t)(FFTK_F_CONV | FFTK_F_TWIDDLE_STORE)) == 0);
        __builtin_assume((p.flags & FFTK_F_CONV) != 0);
        __builtin_assume(p.in_planar == 0);
        __builtin_assume(p.out_planar == 0);
        __builtin_assume(p.stage_io == 0);
        __builtin_assume(p.w_inner == 0);
        __builtin_assume(p.n_in == (uint32_t)Cfg::N);
        __builtin_assume(p.n_out == (uint32_t)Cfg::N);
        __builtin_assume(p.in_nt == 0);
        __builtin_assume(p.out_nt == 0);
    }
    else if constexpr(MODE == 2)
    {
        // (the nontemporal accesses exist in the variants for plain and twiddled passes only)
        __builtin_assume(p.in_nt == 0);
        __builtin_assume(p.out_nt == 0);
    }
    else if constexpr(MODE == 3)
    {
        __builtin_assume(p.load_op == FFTK_LOAD_COMPLEX);
        __builtin_assume(p.store_op == FFTK_STORE_COMPLEX);
        __builtin_assume(p.in_planar == 0);
        __builtin_assume(p.out_planar == 0);
        __builtin_assume(p.stage_io == 0);
        __builtin_assume(p.w_inner == 0);
        __builtin_assume(p.n_in == (uint32_t)Cfg::N);
        __builtin_assume(p.n_out == (uint32_t)Cfg::N);
        __builtin_assume((p.flags & ~(uint32_t)FFTK_F_SCALE) == 0);
        __builtin_assume(p.aux_dim == 0);
        __builtin_assume(p.oc0_first == 0);
    }
}

// Which variants request the table values of the large twiddle on the store side before their
// data: those with registers to spare for them.  The variant for twiddled passes does so for
// powers of two (7 table values at most; the other lengths run other kinds of passes on this
// variant as well, the tile copy of short transforms among them, and the registers the early
// values hold cost those an occupancy step: 100 points went from 63 to 100 registers, 17 points
// spilled).  Double-precision kernels hold 64 registers of data and 60 of pass twiddles; the 7
// table values (28 registers) fit into the first pass of a chirp-z transform up to 512 points,
// beyond that the kernels spill.
template <typename T, typename Cfg, int MODE>
constexpr bool fast_early_twiddles()
{
    constexpr bool pow2 = (Cfg::N & (Cfg::N - 1)) == 0;
    return (MODE == 4 && pow2) || ((MODE == 7 || MODE == 9) && (sizeof(T) == 4 || (MODE == 7 && Cfg::N <= 512)));
}

template <typename T, typename Cfg, int MODE>
__global__ __launch_bounds__(fast_block_limit<Cfg>()) void fast_tile_kernel(const fftk_params p)
{
    typedef typename cplx_of<T>::type C;
    extern __shared__ double2         smem_raw[];
    fast_assume_plain<Cfg, MODE>(p);
    fast_tile_body<T, Cfg, MODE != 0, MODE >= 2, MODE == 4 && sizeof(T) == 4, fast_early_twiddles<T, Cfg, MODE>()>(p, reinterpret_cast<C*>(smem_raw));
}

// The same kernel held to the registers that let WAVES waves share a SIMD.
template <typename T, typename Cfg, int MODE, int WAVES>
__global__ __launch_bounds__(fast_block_limit<Cfg>(), WAVES) void fast_tile_kernel_waves(const fftk_params p)
{
    typedef typename cplx_of<T>::type C;
    extern __shared__ double2         smem_raw[];
    fast_assume_plain<Cfg, MODE>(p);
    fast_tile_body<T, Cfg, MODE != 0, MODE >= 2, MODE == 4 && sizeof(T) == 4, fast_early_twiddles<T, Cfg, MODE>()>(p, reinterpret_cast<C*>(smem_raw));
}

// Waves per SIMD a kernel is compiled for; 0 = whatever its natural register count gives.
// The single-precision variants 3 to 5 are built for four waves (128 registers): their LDS tiles
// (about 33 KB) allow four workgroups a compute unit, and most of them fit without spilling (the
// 4096-point plain kernel: 126 registers; a batch of 1024 on 256 compute units needs four
// workgroups a unit to run in one round).  The full lean kernel keeps its natural count (129-160
// registers for 265 lengths): held to 128 it spills 12-140 bytes a lane, and the passes that
// still run on it (chirp-z, planar, odd-length real, folded tiles) measured the same either way.
template <typename T, typename Cfg, int MODE>
constexpr int fast_waves()
{
    return (sizeof(T) == 4 && (MODE == 3 || MODE == 4 || MODE == 5) && Cfg::TPT <= 512) ? 4 : 0;
}

template <typename T, typename Cfg, int MODE>
int launch_fast(const fftk_params* p, uint32_t grid, size_t lds_bytes, void* stream)
{
    void (*kernel)(const fftk_params);
    if constexpr(fast_waves<T, Cfg, MODE>() != 0)
        kernel = fast_tile_kernel_waves<T, Cfg, MODE, fast_waves<T, Cfg, MODE>()>;
    else
        kernel = fast_tile_kernel<T, Cfg, MODE>;
    if(lds_bytes > 64 * 1024)
    {
        static FftLdsLimit limit;
        if(int rc = limit.allow(kernel))
            return rc;
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(p->nthreads), lds_bytes, (hipStream_t)stream, *p);
    return (int)hipGetLastError();
}

// Variant 4 exists in single precision up to 4096 points (where the registers it saves lift the
// number of waves, and where half-precision arrays are taken in place: the longer kernels
// seldom run such passes, and every variant costs build time).  The variants 0 and 1 exist for
// the lengths marked all_modes.
template <typename T, typename Cfg, int MODE, bool WANTED>
constexpr fast_launch_fn fast_variant()
{
    if constexpr(WANTED)
        return &launch_fast<T, Cfg, MODE>;
    else
        return nullptr;
}

// the table entry of one kernel family, or an empty entry (n = 0) in the translation units
// that do not instantiate it
template <int SLICE, typename T, int PRECISION, int ALL_MODES, bool EXISTS, typename Cfg>
constexpr FastEntry fast_entry()
{
    if constexpr(SLICE == FAST_SLICE && EXISTS)
    {
        constexpr bool more = Cfg::N <= 4096 && sizeof(T) == 4;
        return FastEntry{PRECISION,
                         (uint32_t)Cfg::N,
                         {(uint32_t)Cfg::R0, (uint32_t)Cfg::R1, (uint32_t)Cfg::R2, (uint32_t)Cfg::R3},
                         (uint32_t)Cfg::TPT,
                         &launch_fast<T, Cfg, 2>,
                         fast_variant<T, Cfg, 1, ALL_MODES != 0>(),
                         fast_variant<T, Cfg, 0, ALL_MODES != 0>(),
                         &launch_fast<T, Cfg, 3>,
                         fast_variant<T, Cfg, 4, more>(),
                         fast_variant<T, Cfg, 5, Cfg::N % 2 == 1 && (Cfg::N > 1)>(),
                         fast_variant<T, Cfg, 7, ALL_MODES != 0>(),
                         fast_variant<T, Cfg, 8, ALL_MODES != 0>(),
                         fast_variant<T, Cfg, 9, ALL_MODES != 0>()};
    }
    else
        return FastEntry{-1, 0, {1, 1, 1, 1}, 0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
}

#define FAST_SCHED(SLICE, FULL, N, A, B, C, D, TTF, TTD, DBL)                  \
    fast_entry<SLICE, float, 0, FULL, true, FastCfg<N, A, B, C, D, TTF>>(),     \
        fast_entry<SLICE, double, 1, FULL, (DBL) != 0, FastCfg<N, A, B, C, D, (DBL) ? TTD : TTF>>(),

// (a build for experiments may name a shorter list: -DFAST_SCHEDULES_FILE='"..."')
#ifndef FAST_SCHEDULES_FILE
#define FAST_SCHEDULES_FILE "fast_schedules.h"
#endif
const FastEntry g_slice[] = {
#include FAST_SCHEDULES_FILE
};
static_assert(FAST_SLICE >= 0 && FAST_SLICE < FAST_SLICES, "compile with -DFAST_SLICE=0..FAST_SLICES-1");

} // namespace

#define FAST_SLICE_FN2(I) fftrt_fast_slice_##I
#define FAST_SLICE_FN(I) FAST_SLICE_FN2(I)

extern "C" const FastEntry* FAST_SLICE_FN(FAST_SLICE)(int* count)
{
    *count = (int)(sizeof(g_slice) / sizeof(g_slice[0]));
    return g_slice;
}

#if FAST_SLICE == 0
#define FAST_SLICE_LIST(X)                                                                              \
    X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14) X(15) X(16) X(17) X(18) \
        X(19) X(20) X(21) X(22) X(23)
static_assert(FAST_SLICES == 24, "FAST_SLICE_LIST names twenty-four slices");
#define FAST_DECLARE(I) extern "C" const FastEntry* fftrt_fast_slice_##I(int*);
FAST_SLICE_LIST(FAST_DECLARE)

namespace
{

// All entries, sorted by (precision, n).  The list normally holds one schedule per length;
// a tuning build may hold several, and ROCFFT_AMD_FAST_VARIANT=<v> then selects the
// (v mod count)-th of each length.
const std::vector<const FastEntry*>& fast_index()
{
    static std::vector<const FastEntry*> index;
    static std::once_flag                once;
    std::call_once(once, []() {
        typedef const FastEntry* (*slice_fn)(int*);
#define FAST_NAME(I) fftrt_fast_slice_##I,
        const slice_fn slices[FAST_SLICES] = {FAST_SLICE_LIST(FAST_NAME)};
        for(slice_fn f : slices)
        {
            int              cnt = 0;
            const FastEntry* e   = f(&cnt);
            for(int i = 0; i < cnt; ++i)
                if(e[i].n != 0) // (empty: instantiated in another slice, or no such kernel)
                    index.push_back(e + i);
        }
        std::stable_sort(index.begin(), index.end(), [](const FastEntry* a, const FastEntry* b) {
            return a->precision != b->precision ? a->precision < b->precision : a->n < b->n;
        });
        const char*  env     = getenv("ROCFFT_AMD_FAST_VARIANT");
        const size_t variant = env ? (size_t)strtoul(env, nullptr, 10) : 0;
        std::vector<const FastEntry*> picked;
        for(size_t i = 0; i < index.size();)
        {
            size_t j = i;
            while(j < index.size() && index[j]->precision == index[i]->precision && index[j]->n == index[i]->n)
                ++j;
            picked.push_back(index[i + variant % (j - i)]);
            i = j;
        }
        index.swap(picked);
    });
    return index;
}

const FastEntry* find_fast(int precision, uint32_t n)
{
    const auto& index = fast_index();
    auto        it    = std::lower_bound(index.begin(), index.end(), n, [&](const FastEntry* e, uint32_t v) {
        return e->precision != precision ? e->precision < precision : e->n < v;
    });
    if(it == index.end() || (*it)->precision != precision || (*it)->n != n)
        return nullptr;
    return *it;
}

} // namespace

extern "C" uint32_t fftrt_fast_schedule(int precision, uint32_t n, uint32_t* radix, uint32_t* nf)
{
    const FastEntry* e = find_fast(precision, n);
    if(!e)
        return 0;
    uint32_t cnt = 0;
    for(uint32_t i = 0; i < 4; ++i)
        if(e->radix[i] > 1)
            radix[cnt++] = e->radix[i];
    *nf = cnt;
    return e->tpt;
}

// is there a compiled kernel of this length that reads or writes half-precision arrays?
extern "C" int fftrt_fast_takes_half(uint32_t n)
{
    const FastEntry* e = find_fast(0, n);
    return e && e->more ? 1 : 0;
}

// called by fftrt_launch_tile (kernels.hip) when the plan asked for the fast kernel;
// returns FFTRT_NO_FAST_VARIANT when this access mode has no compiled variant
extern "C" int fftrt_launch_fast_tile(const struct fftk_params* p, int precision, int vec, uint32_t grid,
                                      size_t lds_bytes, void* stream)
{
    const FastEntry* e = find_fast(precision, p->n);
    if(!e || p->T != e->tpt || p->nthreads > (e->tpt > 512 ? 1024u : 512u) || p->padshift != 4)
        return (int)hipErrorInvalidValue;
    uint32_t cnt = 0;
    for(uint32_t i = 0; i < 4; ++i)
        if(e->radix[i] > 1 && (cnt >= p->nf || p->radix[cnt++] != e->radix[i]))
            return (int)hipErrorInvalidValue;
    if(cnt != p->nf)
        return (int)hipErrorInvalidValue;
    fast_launch_fn fn = p->lean ? e->lean : vec ? e->vec : e->scalar;
    if(p->in_half || p->out_half)
    {
        // (the planner offers such passes only after fftrt_fast_takes_half said yes)
        if(!p->lean || !e->more)
            return (int)hipErrorInvalidValue;
        return e->more(p, grid, lds_bytes, stream);
    }
    // the variants compiled for some kinds of passes alone (see fast_assume_plain);
    // ROCFFT_AMD_NO_VARIANTS=1 keeps every pass on the full lean kernel (for comparisons)
    static const bool variants = !getenv("ROCFFT_AMD_NO_VARIANTS");
    if(variants && p->lean && !p->in_planar && !p->out_planar && !p->w_inner)
    {
        const bool plain_ops = p->load_op == FFTK_LOAD_COMPLEX && p->store_op == FFTK_STORE_COMPLEX && !p->stage_io
                               && p->n_in == p->n && p->n_out == p->n;
        const bool only_scale = (p->flags & ~(uint32_t)FFTK_F_SCALE) == 0 && p->aux_dim == 0 && !p->oc0_first;
        if(plain_ops && only_scale)
            fn = e->plain;
        else if(e->more && (p->flags & ~(uint32_t)(FFTK_F_SCALE | FFTK_F_TWIDDLE_STORE)) == 0
                && (p->load_op == FFTK_LOAD_COMPLEX || p->load_op == FFTK_LOAD_C2R_PRE)
                && (p->store_op == FFTK_STORE_COMPLEX || p->store_op == FFTK_STORE_R2C_POST))
            fn = e->more;
        else if(e->odd_real && only_scale && !p->stage_io
                && ((p->load_op == FFTK_LOAD_REAL && p->store_op == FFTK_STORE_COMPLEX)
                    || (p->load_op == FFTK_LOAD_HERM_EXPAND && p->store_op == FFTK_STORE_REAL)))
            fn = e->odd_real;
    }
    // the first and last pass of a chirp-z transform in three kernels (kernels of their own, so
    // that a profile tells them apart)
    if(variants && p->lean && !p->in_planar && !p->out_planar && !p->w_inner && !p->stage_io
       && p->load_op == FFTK_LOAD_COMPLEX && p->store_op == FFTK_STORE_COMPLEX)
    {
        if(e->chirp_in && (p->flags & FFTK_F_CHIRP_LOAD)
           && (p->flags & ~(uint32_t)(FFTK_F_CHIRP_LOAD | FFTK_F_TWIDDLE_STORE | FFTK_F_CHIRP_CONJ)) == 0)
            fn = e->chirp_in;
        else if(e->chirp_out && (p->flags & FFTK_F_CHIRP_STORE) && p->n_in == p->n
                && (p->flags & ~(uint32_t)(FFTK_F_CHIRP_STORE | FFTK_F_SCALE | FFTK_F_CHIRP_CONJ)) == 0)
            fn = e->chirp_out;
        else if(e->chirp_mid && (p->flags & FFTK_F_CONV) && p->n_in == p->n && p->n_out == p->n
                && (p->flags & ~(uint32_t)(FFTK_F_CONV | FFTK_F_TWIDDLE_STORE)) == 0)
            fn = e->chirp_mid;
    }
    if(!fn)
        return FFTRT_NO_FAST_VARIANT;
    fftk_params without_nt;
    if((p->in_nt || p->out_nt) && fn != e->plain && fn != e->more)
    {
        without_nt        = *p;
        without_nt.in_nt  = 0;
        without_nt.out_nt = 0;
        p                 = &without_nt;
    }
    return fn(p, grid, lds_bytes, stream);
}
#endif
