// tile_core.h -- the phases of the tile FFT kernel, written against explicit
// (block id, thread id) arguments so that the HIP kernel and the host-side
// emulation used by the CPU tests share one body.
//
// Phases of one workgroup (barriers between them are the caller's job):
//   tile_load   global -> LDS, with the fused input operation
//   pass_read   LDS -> registers for one Stockham pass
//   pass_write  twiddle, butterfly, registers -> LDS (autosort positions)
//   tile_conv   (convolution mode) multiply by a spectrum between two FFTs
//   tile_store  LDS -> global, with the fused output operation
//
// Stockham indexing follows the reference's in-LDS autosort
// (library/src/device/generator/stockham_gen_base.h:347-456): butterfly b of a
// radix-w pass with cumulative height c reads A[b + k*n/w] and writes
// A[(b div c)*w*c + (b mod c) + k*c].  The twiddle table layout is this
// library's own: pass p stores e^{-2 pi i jk/(c w)} at twoff[p] + (k-1)*c + j.
#ifndef ROCFFT_AMD_TILE_CORE_H
#define ROCFFT_AMD_TILE_CORE_H

#include "butterfly.h"
#include "kparams.h"

template <typename T>
struct TileCtx
{
    uint32_t tile0;    // first tile-dimension index of this workgroup
    uint32_t oi[3];    // outer indices
    int64_t  ibase;    // input scalar offset of (j=0, w=0)
    int64_t  obase;    // output scalar offset of (j=0, w=0)
    uint32_t q_block;  // auxiliary index when it is uniform over the workgroup
    uint32_t b0;       // folded tile axis: second-axis index of the workgroup's first tile entry
};

// scalar offset of tile entry w of the workgroup from ibase / obase
template <typename T>
FFT_DEV int64_t tile_w_in(const fftk_params& p, const TileCtx<T>& c, uint32_t w)
{
    if(!p.w_inner)
        return (int64_t)w * p.w_is;
    const uint32_t g = c.tile0 + w, b = g / p.w_inner;
    return (int64_t)(b - c.b0) * p.w2_is + (int64_t)(g - b * p.w_inner) * p.w_is;
}
template <typename T>
FFT_DEV int64_t tile_w_out(const fftk_params& p, const TileCtx<T>& c, uint32_t w)
{
    if(!p.w_inner)
        return (int64_t)w * p.w_os;
    const uint32_t g = c.tile0 + w, b = g / p.w_inner;
    return (int64_t)(b - c.b0) * p.w2_os + (int64_t)(g - b * p.w_inner) * p.w_os;
}

template <typename T>
FFT_DEV void tile_decode(const fftk_params& p, uint32_t bid, TileCtx<T>& c)
{
    if(p.xcd_remap)
    {
        // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Renumber so
        // that every XCD works through one contiguous range of tiles: neighbouring tiles,
        // which share cache lines and DRAM pages, then meet in the same L2 at the same time.
        const uint32_t grid = p.grid, xcd = bid & 7u, idx = bid >> 3;
        const uint32_t qd = grid >> 3, rm = grid & 7u;
        bid = xcd * qd + (xcd < rm ? xcd : rm) + idx;
    }
    uint32_t ntile = (p.tile_cnt + p.W - 1) >> p.wshift;
    uint32_t tb;
    if(p.oc0_first)
    {
        // workgroups that differ in outer index 0 only (the signals of a batch) are neighbours:
        // they read the same rows of a chirp or spectrum table, one after the other in one L2
        c.oi[0] = bid % p.oc[0];
        bid /= p.oc[0];
        tb = bid % ntile;
        bid /= ntile;
    }
    else
    {
        tb = bid % ntile;
        bid /= ntile;
        c.oi[0] = bid % p.oc[0];
        bid /= p.oc[0];
    }
    c.oi[1] = bid % p.oc[1];
    c.oi[2] = bid / p.oc[1];
    c.tile0 = tb << p.wshift;
    c.b0    = p.w_inner ? c.tile0 / p.w_inner : 0;
    // folded tile axis: the bases point at entry (0, b0), the per-entry offsets count from there
    c.ibase = (p.w_inner ? (int64_t)c.b0 * p.w2_is : (int64_t)c.tile0 * p.w_is) + (int64_t)c.oi[0] * p.o_is[0]
              + (int64_t)c.oi[1] * p.o_is[1] + (int64_t)c.oi[2] * p.o_is[2];
    c.obase = (p.w_inner ? (int64_t)c.b0 * p.w2_os : (int64_t)c.tile0 * p.w_os) + (int64_t)c.oi[0] * p.o_os[0]
              + (int64_t)c.oi[1] * p.o_os[1] + (int64_t)c.oi[2] * p.o_os[2];
    // (no indexing of oi[] with a run-time value: that would push the context into scratch memory)
    c.q_block = (p.aux_dim == 2 ? c.oi[0] : p.aux_dim == 3 ? c.oi[1] : p.aux_dim == 4 ? c.oi[2] : 0) >> p.aux_shift;
}

FFT_DEV uint32_t lds_addr(const fftk_params& p, uint32_t w, uint32_t j)
{
    return w * p.pitch + j + (j >> p.padshift);
}

// ---- user callbacks.  `off` counts scalars from the kernel's base pointer of that side.
template <typename T>
FFT_DEV T cb_load_scalar(const fftk_cb& cb, int64_t off)
{
    typedef T (*fn_t)(T*, size_t, void*, void*);
    return reinterpret_cast<fn_t>(const_cast<void*>(cb.load_fn))(
        static_cast<T*>(const_cast<void*>(cb.in_base)), (size_t)(cb.in_off + off), cb.load_data, nullptr);
}
template <typename T>
FFT_DEV typename cplx_of<T>::type cb_load_pair(const fftk_cb& cb, int64_t off)
{
    typedef typename cplx_of<T>::type C;
    typedef C (*fn_t)(C*, size_t, void*, void*);
    return reinterpret_cast<fn_t>(const_cast<void*>(cb.load_fn))(
        static_cast<C*>(const_cast<void*>(cb.in_base)), (size_t)((cb.in_off + off) >> 1), cb.load_data, nullptr);
}
template <typename T>
FFT_DEV void cb_store_scalar(const fftk_cb& cb, int64_t off, T v)
{
    typedef void (*fn_t)(T*, size_t, T, void*, void*);
    reinterpret_cast<fn_t>(const_cast<void*>(cb.store_fn))(static_cast<T*>(cb.out_base), (size_t)(cb.out_off + off), v,
                                                            cb.store_data, nullptr);
}
template <typename T>
FFT_DEV void cb_store_pair(const fftk_cb& cb, int64_t off, typename cplx_of<T>::type v)
{
    typedef typename cplx_of<T>::type C;
    typedef void (*fn_t)(C*, size_t, C, void*, void*);
    reinterpret_cast<fn_t>(const_cast<void*>(cb.store_fn))(static_cast<C*>(cb.out_base), (size_t)((cb.out_off + off) >> 1), v,
                                                            cb.store_data, nullptr);
}
// One element whose parts lie at re0[off] and im0[off] (im0 = re0 + a few scalars for
// interleaved and real-pair layouts), through the load callback when there is one.
template <typename T>
FFT_DEV typename cplx_of<T>::type cb_or_load(const fftk_cb& cb, const T* re0, const T* im0, int64_t off)
{
    typename cplx_of<T>::type v;
    if(cb.load_fn)
    {
        if(cb.in_complex)
            return cb_load_pair<T>(cb, off);
        v.x = cb_load_scalar<T>(cb, off);
        v.y = cb_load_scalar<T>(cb, off + (im0 - re0));
        return v;
    }
    v.x = re0[off];
    v.y = im0[off];
    return v;
}
template <typename T>
FFT_DEV void cb_or_store(const fftk_cb& cb, T* re0, T* im0, int64_t off, typename cplx_of<T>::type v)
{
    if(cb.store_fn)
    {
        if(cb.out_complex)
            cb_store_pair<T>(cb, off, v);
        else
        {
            cb_store_scalar<T>(cb, off, v.x);
            cb_store_scalar<T>(cb, off + (im0 - re0), v.y);
        }
        return;
    }
    re0[off] = v.x;
    im0[off] = v.y;
}

template <typename T, bool VEC>
FFT_DEV typename cplx_of<T>::type load_elem(const fftk_params& p, int64_t off)
{
    typedef typename cplx_of<T>::type C;
    if(p.cb.load_fn)
        return cb_or_load<T>(p.cb, static_cast<const T*>(p.in0), static_cast<const T*>(p.in1), off);
    C v;
    if(VEC)
        v = *reinterpret_cast<const C*>(static_cast<const T*>(p.in0) + off);
    else
    {
        v.x = static_cast<const T*>(p.in0)[off];
        v.y = static_cast<const T*>(p.in1)[off];
    }
    return v;
}

template <typename T, bool VEC>
FFT_DEV void store_elem(const fftk_params& p, int64_t off, typename cplx_of<T>::type v)
{
    typedef typename cplx_of<T>::type C;
    if(p.cb.store_fn)
    {
        cb_or_store<T>(p.cb, static_cast<T*>(p.out0), static_cast<T*>(p.out1), off, v);
        return;
    }
    if(VEC)
        *reinterpret_cast<C*>(static_cast<T*>(p.out0) + off) = v;
    else
    {
        static_cast<T*>(p.out0)[off] = v.x;
        static_cast<T*>(p.out1)[off] = v.y;
    }
}

// Walks (w, j) over W x jcount, fastest along the tile dimension when
// `fast_tile`, else along the transform; calls f(w, j).
template <typename F>
FFT_DEV void tile_walk(const fftk_params& p, uint32_t tid, uint32_t jcount, bool fast_tile, F f)
{
    if(fast_tile)
    {
        uint32_t w  = tid & (p.W - 1);
        uint32_t dj = p.nthreads >> p.wshift;
        for(uint32_t j = tid >> p.wshift; j < jcount; j += dj)
            f(w, j);
    }
    else
    {
        uint32_t j = tid % jcount;
        uint32_t w = tid / jcount;
        while(w < p.W)
        {
            f(w, j);
            j += p.nthreads;
            while(j >= jcount)
            {
                j -= jcount;
                ++w;
            }
        }
    }
}

// One logical input element (tile transform w, position j) with the fused input
// operation applied, ready for the forward butterflies (re/im exchanged when the
// pass is an inverse transform).  Not used by the C2R pre-processing load.
template <typename T, bool VEC>
FFT_DEV typename cplx_of<T>::type
    fetch_elem(const fftk_params& p, const TileCtx<T>& c, uint32_t w, uint32_t j)
{
    typedef typename cplx_of<T>::type C;
    C                                 v;
    v.x = 0;
    v.y = 0;
    bool     ok  = (c.tile0 + w < p.tile_cnt) && (j < p.n_in);
    uint32_t idx = 0;
    if(ok && (p.flags & FFTK_F_CHIRP_LOAD))
    {
        uint32_t q = p.aux_dim == 1 ? (c.tile0 + w) >> p.aux_shift : c.q_block;
        idx        = j * p.chirp_js + q * p.chirp_qs;
        ok         = idx < p.blu_n;
    }
    if(ok)
    {
        int64_t base = c.ibase + tile_w_in<T>(p, c, w);
        if(p.load_op == FFTK_LOAD_REAL)
            v.x = p.cb.load_fn ? cb_load_scalar<T>(p.cb, base + (int64_t)j * p.t_is)
                               : static_cast<const T*>(p.in0)[base + (int64_t)j * p.t_is];
        else if(p.load_op == FFTK_LOAD_HERM_EXPAND)
        {
            // logical length n_in; bins above n_in/2 are the conjugate mirror,
            // imaginary parts of bin 0 and of the Nyquist bin are ignored
            uint32_t jm = j <= p.n_in / 2 ? j : p.n_in - j;
            v           = load_elem<T, VEC>(p, base + (int64_t)jm * p.t_is);
            if(jm != j)
                v.y = -v.y;
            if(j == 0 || 2 * j == p.n_in)
                v.y = 0;
        }
        else
            v = load_elem<T, VEC>(p, base + (int64_t)j * p.t_is);
        if(p.flags & FFTK_F_CHIRP_LOAD)
        {
            C ch = static_cast<const C*>(p.chirp)[idx];
            v    = (p.flags & FFTK_F_CHIRP_CONJ) ? c_mul(v, ch) : c_mulc(v, ch);
        }
    }
    return p.dir > 0 ? c_swap(v) : v;
}

template <typename T, bool VEC>
FFT_DEV void tile_load(const fftk_params&           p,
                       const TileCtx<T>&            c,
                       typename cplx_of<T>::type*   lds,
                       uint32_t                     tid)
{
    typedef typename cplx_of<T>::type C;
    const bool                        inv = p.dir > 0;
    if(p.load_op != FFTK_LOAD_C2R_PRE)
    {
        tile_walk(p, tid, p.n, p.in_fast_tile != 0, [&](uint32_t w, uint32_t j) {
            lds[lds_addr(p, w, j)] = fetch_elem<T, VEC>(p, c, w, j);
        });
    }
    else
    {
        // reference math: library/src/device/kernels/real2complex_device.h:212-254
        const uint32_t n = p.n;
        tile_walk(p, tid, n / 2 + 1, p.in_fast_tile != 0, [&](uint32_t w, uint32_t j) {
            bool    ok   = c.tile0 + w < p.tile_cnt;
            int64_t base = c.ibase + tile_w_in<T>(p, c, w);
            C       zj, zq;
            zj.x = zj.y = zq.x = zq.y = 0;
            uint32_t jq              = n - j;
            if(ok)
            {
                C a = load_elem<T, VEC>(p, base + (int64_t)j * p.t_is);
                if(j == 0)
                {
                    C b  = load_elem<T, VEC>(p, base + (int64_t)n * p.t_is);
                    zj.x = a.x + b.x;
                    zj.y = a.x - b.x;
                }
                else if(j == jq)
                {
                    zj.x = (T)2 * a.x;
                    zj.y = (T)-2 * a.y;
                }
                else
                {
                    C b  = load_elem<T, VEC>(p, base + (int64_t)jq * p.t_is);
                    C u  = c_add(a, b);
                    C v  = c_sub(a, b);
                    C t  = static_cast<const C*>(p.half_tw)[j];
                    zj.x = u.x + v.x * t.y - u.y * t.x;
                    zj.y = v.y + u.y * t.y + v.x * t.x;
                    zq.x = u.x - v.x * t.y + u.y * t.x;
                    zq.y = -v.y + u.y * t.y + v.x * t.x;
                }
            }
            lds[lds_addr(p, w, j)] = inv ? c_swap(zj) : zj;
            if(j != 0 && j != jq)
                lds[lds_addr(p, w, jq)] = inv ? c_swap(zq) : zq;
        });
    }
}

// thread -> (transform of the tile, lane within the transform)
FFT_DEV void thread_role(const fftk_params& p, uint32_t tid, uint32_t& w, uint32_t& tt, bool& active)
{
    active = tid < p.T * p.W;
    if(p.wfast)
    {
        w  = tid & (p.W - 1);
        tt = tid >> p.wshift;
    }
    else
    {
        tt = tid % p.T;
        w  = tid / p.T;
    }
}

template <typename T, int R>
FFT_DEV void pass_read(const fftk_params&               p,
                       const typename cplx_of<T>::type* lds,
                       uint32_t                         w,
                       uint32_t                         tt,
                       bool                             active,
                       typename cplx_of<T>::type*       r)
{
    constexpr int  MAXS = FFTK_REG_ELEMS / R;
    const uint32_t m    = p.n / R;
#pragma unroll
    for(int s = 0; s < MAXS; ++s)
    {
        uint32_t b = tt + s * p.T;
        if(active && b < m)
        {
#pragma unroll
            for(int k = 0; k < R; ++k)
                r[s * R + k] = lds[lds_addr(p, w, b + k * m)];
        }
    }
}

template <typename T, int R>
FFT_DEV void pass_write(const fftk_params&         p,
                        int                        pass,
                        typename cplx_of<T>::type* lds,
                        uint32_t                   w,
                        uint32_t                   tt,
                        bool                       active,
                        typename cplx_of<T>::type* r)
{
    typedef typename cplx_of<T>::type C;
    constexpr int                     MAXS = FFTK_REG_ELEMS / R;
    const uint32_t                    m    = p.n / R;
    const uint32_t                    c    = p.cum[pass];
    const uint32_t                    sh   = p.cshift[pass];
    const C*                          tw   = static_cast<const C*>(p.tw) + p.twoff[pass];
#pragma unroll
    for(int s = 0; s < MAXS; ++s)
    {
        uint32_t b = tt + s * p.T;
        if(active && b < m)
        {
            uint32_t bl, bh;
            if(sh != 0xff)
            {
                bl = b & (c - 1);
                bh = b >> sh;
            }
            else
            {
                bh = b / c;
                bl = b - bh * c;
            }
            if(c > 1)
            {
#pragma unroll
                for(int k = 1; k < R; ++k)
                    r[s * R + k] = c_mul(r[s * R + k], tw[(k - 1) * c + bl]);
            }
            Butterfly<T, R>::run(r + s * R);
            uint32_t o = bh * R * c + bl;
#pragma unroll
            for(int k = 0; k < R; ++k)
                lds[lds_addr(p, w, o + k * c)] = r[s * R + k];
        }
    }
}

// convolution mode: data in LDS holds the forward spectrum; multiply it by the
// stored spectrum and exchange re/im so that the next forward run is an inverse FFT
template <typename T>
FFT_DEV void tile_conv(const fftk_params&         p,
                       const TileCtx<T>&          c,
                       typename cplx_of<T>::type* lds,
                       uint32_t                   tid)
{
    typedef typename cplx_of<T>::type C;
    tile_walk(p, tid, p.n, false, [&](uint32_t w, uint32_t j) {
        if(c.tile0 + w >= p.tile_cnt)
            return;
        uint32_t q = p.aux_dim == 1 ? (c.tile0 + w) >> p.aux_shift : c.q_block;
        C        v = lds[lds_addr(p, w, j)];
        C        b = static_cast<const C*>(p.convb)[j + q * p.convb_qs];
        v          = c_mul(v, b);
        lds[lds_addr(p, w, j)] = c_swap(v);
    });
}

template <typename T>
FFT_DEV typename cplx_of<T>::type large_twiddle(const fftk_params& p, uint32_t u)
{
    typedef typename cplx_of<T>::type C;
    const C*                          tbl = static_cast<const C*>(p.ltw);
    C                                 lo  = tbl[u & ((1u << p.ltw_shift) - 1)];
    C                                 hi  = tbl[(1u << p.ltw_shift) + (u >> p.ltw_shift)];
    return c_mul(lo, hi);
}

// Writes one logical output element (tile transform w, position j): undoes the
// re/im exchange of inverse passes, applies the fused output operation, stores.
// Not used by the R2C post-processing store.
template <typename T, bool VEC>
FFT_DEV void emit_elem(const fftk_params& p, const TileCtx<T>& c, uint32_t w, uint32_t j,
                       typename cplx_of<T>::type v)
{
    typedef typename cplx_of<T>::type C;
    // direction of the transform that produced v
    const bool inv = (p.flags & FFTK_F_CONV) ? true : (p.dir > 0);
    if(c.tile0 + w >= p.tile_cnt || j >= p.n_out)
        return;
    if(inv)
        v = c_swap(v);
    uint32_t q = p.aux_dim == 1 ? (c.tile0 + w) >> p.aux_shift : c.q_block;
    if(p.flags & FFTK_F_TWIDDLE_STORE)
    {
        C t = large_twiddle<T>(p, j * (q * p.ltw_qmul + p.ltw_qadd));
        v   = inv ? c_mulc(v, t) : c_mul(v, t);
    }
    if(p.flags & FFTK_F_CHIRP_STORE)
    {
        uint32_t idx = j * p.chirp_js + q * p.chirp_qs;
        if(idx >= p.blu_n)
            return;
        C ch = static_cast<const C*>(p.chirp)[idx];
        v    = (p.flags & FFTK_F_CHIRP_CONJ) ? c_mul(v, ch) : c_mulc(v, ch);
    }
    if(p.flags & FFTK_F_SCALE)
    {
        v.x *= (T)p.scale;
        v.y *= (T)p.scale;
    }
    int64_t off = c.obase + (int64_t)j * p.t_os + tile_w_out<T>(p, c, w);
    if(p.store_op == FFTK_STORE_REAL)
    {
        if(p.cb.store_fn)
            cb_store_scalar<T>(p.cb, off, v.x);
        else
            static_cast<T*>(p.out0)[off] = v.x;
    }
    else
        store_elem<T, VEC>(p, off, v);
}

template <typename T, bool VEC>
FFT_DEV void tile_store(const fftk_params&               p,
                        const TileCtx<T>&                c,
                        const typename cplx_of<T>::type* lds,
                        uint32_t                         tid)
{
    typedef typename cplx_of<T>::type C;
    if(p.store_op == FFTK_STORE_COMPLEX || p.store_op == FFTK_STORE_REAL)
    {
        tile_walk(p, tid, p.n_out, p.out_fast_tile != 0, [&](uint32_t w, uint32_t j) {
            emit_elem<T, VEC>(p, c, w, j, lds[lds_addr(p, w, j)]);
        });
    }
    else // FFTK_STORE_R2C_POST
    {
        // reference math: library/src/device/kernels/real2complex_device.h:25-103
        const uint32_t n = p.n;
        tile_walk(p, tid, n / 2 + 1, p.out_fast_tile != 0, [&](uint32_t w, uint32_t j) {
            if(c.tile0 + w >= p.tile_cnt)
                return;
            int64_t  base = c.obase + tile_w_out<T>(p, c, w);
            uint32_t jq   = n - j;
            C        zp   = lds[lds_addr(p, w, j)];
            C        o0, o1;
            bool     two = true;
            if(j == 0)
            {
                o0.x = zp.x + zp.y;
                o0.y = 0;
                o1.x = zp.x - zp.y;
                o1.y = 0;
            }
            else if(j == jq)
            {
                o0.x = zp.x;
                o0.y = -zp.y;
                two  = false;
            }
            else
            {
                C zq = lds[lds_addr(p, w, jq)];
                C u, v;
                u.x  = (T)0.5 * (zp.x + zq.x);
                u.y  = (T)0.5 * (zp.y + zq.y);
                v.x  = (T)0.5 * (zp.x - zq.x);
                v.y  = (T)0.5 * (zp.y - zq.y);
                C t  = static_cast<const C*>(p.half_tw)[j];
                o0.x = u.x + v.x * t.y + u.y * t.x;
                o0.y = v.y + u.y * t.y - v.x * t.x;
                o1.x = u.x - v.x * t.y - u.y * t.x;
                o1.y = -v.y + u.y * t.y - v.x * t.x;
            }
            if(p.flags & FFTK_F_SCALE)
            {
                o0.x *= (T)p.scale;
                o0.y *= (T)p.scale;
                o1.x *= (T)p.scale;
                o1.y *= (T)p.scale;
            }
            store_elem<T, VEC>(p, base + (int64_t)j * p.t_os, o0);
            if(two)
                store_elem<T, VEC>(p, base + (int64_t)jq * p.t_os, o1);
        });
    }
}

// ---------------------------------------------------------------------------
// standalone even-length real post-/pre-processing on natural-order rows
// (used when the half-length complex FFT does not fit one kernel)

template <typename T>
FFT_DEV void real_post_elem(const fftk_real_params& p, uint64_t gid)
{
    typedef typename cplx_of<T>::type C;
    const uint32_t                    L  = p.half;
    const uint32_t                    jc = L / 2 + 1;
    uint32_t                          j  = (uint32_t)(gid % jc);
    uint64_t                          r  = gid / jc;
    uint32_t                          r0 = (uint32_t)(r % p.rows0);
    r /= p.rows0;
    uint32_t r1 = (uint32_t)(r % p.rows1);
    uint32_t r2 = (uint32_t)(r / p.rows1);
    if(r2 >= p.rows2)
        return;
    const T* z0 = static_cast<const T*>(p.z0);
    const T* z1 = static_cast<const T*>(p.z1);
    T*       h0 = static_cast<T*>(p.ho0);
    T*       h1 = static_cast<T*>(p.ho1);
    int64_t  zb = (int64_t)r0 * p.z_r0 + (int64_t)r1 * p.z_r1 + (int64_t)r2 * p.z_r2;
    int64_t  hb = (int64_t)r0 * p.h_r0 + (int64_t)r1 * p.h_r1 + (int64_t)r2 * p.h_r2;
    uint32_t jq = L - j;
    C        zp;
    zp.x = z0[zb + (int64_t)j * p.z_s];
    zp.y = z1[zb + (int64_t)j * p.z_s];
    C    o0, o1;
    bool two = true;
    if(j == 0)
    {
        o0.x = zp.x + zp.y;
        o0.y = 0;
        o1.x = zp.x - zp.y;
        o1.y = 0;
    }
    else if(j == jq)
    {
        o0.x = zp.x;
        o0.y = -zp.y;
        two  = false;
    }
    else
    {
        C zq;
        zq.x = z0[zb + (int64_t)jq * p.z_s];
        zq.y = z1[zb + (int64_t)jq * p.z_s];
        C u, v;
        u.x  = (T)0.5 * (zp.x + zq.x);
        u.y  = (T)0.5 * (zp.y + zq.y);
        v.x  = (T)0.5 * (zp.x - zq.x);
        v.y  = (T)0.5 * (zp.y - zq.y);
        C t  = static_cast<const C*>(p.half_tw)[j];
        o0.x = u.x + v.x * t.y + u.y * t.x;
        o0.y = v.y + u.y * t.y - v.x * t.x;
        o1.x = u.x - v.x * t.y - u.y * t.x;
        o1.y = -v.y + u.y * t.y - v.x * t.x;
    }
    if(p.use_scale)
    {
        o0.x *= (T)p.scale;
        o0.y *= (T)p.scale;
        o1.x *= (T)p.scale;
        o1.y *= (T)p.scale;
    }
    cb_or_store<T>(p.cb, h0, h1, hb + (int64_t)j * p.h_s, o0);
    if(two)
        cb_or_store<T>(p.cb, h0, h1, hb + (int64_t)jq * p.h_s, o1);
}

template <typename T>
FFT_DEV void real_pre_elem(const fftk_real_params& p, uint64_t gid)
{
    typedef typename cplx_of<T>::type C;
    const uint32_t                    L  = p.half;
    const uint32_t                    jc = L / 2 + 1;
    uint32_t                          j  = (uint32_t)(gid % jc);
    uint64_t                          r  = gid / jc;
    uint32_t                          r0 = (uint32_t)(r % p.rows0);
    r /= p.rows0;
    uint32_t r1 = (uint32_t)(r % p.rows1);
    uint32_t r2 = (uint32_t)(r / p.rows1);
    if(r2 >= p.rows2)
        return;
    const T* h0 = static_cast<const T*>(p.h0);
    const T* h1 = static_cast<const T*>(p.h1);
    T*       z0 = static_cast<T*>(p.zo0);
    T*       z1 = static_cast<T*>(p.zo1);
    int64_t  zb = (int64_t)r0 * p.z_r0 + (int64_t)r1 * p.z_r1 + (int64_t)r2 * p.z_r2;
    int64_t  hb = (int64_t)r0 * p.h_r0 + (int64_t)r1 * p.h_r1 + (int64_t)r2 * p.h_r2;
    uint32_t jq = L - j;
    C        a   = cb_or_load<T>(p.cb, h0, h1, hb + (int64_t)j * p.h_s);
    C        zj, zq;
    bool     two = true;
    zq.x = zq.y = 0;
    if(j == 0)
    {
        T bx = cb_or_load<T>(p.cb, h0, h1, hb + (int64_t)L * p.h_s).x;
        zj.x = a.x + bx;
        zj.y = a.x - bx;
        two  = false;
    }
    else if(j == jq)
    {
        zj.x = (T)2 * a.x;
        zj.y = (T)-2 * a.y;
        two  = false;
    }
    else
    {
        C b  = cb_or_load<T>(p.cb, h0, h1, hb + (int64_t)jq * p.h_s);
        C u  = c_add(a, b);
        C v  = c_sub(a, b);
        C t  = static_cast<const C*>(p.half_tw)[j];
        zj.x = u.x + v.x * t.y - u.y * t.x;
        zj.y = v.y + u.y * t.y + v.x * t.x;
        zq.x = u.x - v.x * t.y + u.y * t.x;
        zq.y = -v.y + u.y * t.y + v.x * t.x;
    }
    if(p.use_scale)
    {
        zj.x *= (T)p.scale;
        zj.y *= (T)p.scale;
    }
    z0[zb + (int64_t)j * p.z_s] = zj.x;
    z1[zb + (int64_t)j * p.z_s] = zj.y;
    if(two)
    {
        if(p.use_scale)
        {
            zq.x *= (T)p.scale;
            zq.y *= (T)p.scale;
        }
        z0[zb + (int64_t)jq * p.z_s] = zq.x;
        z1[zb + (int64_t)jq * p.z_s] = zq.y;
    }
}

// half-precision storage types of the staging copies
typedef _Float16 fft_half;
struct fft_half2
{
    _Float16 x, y;
};
FFT_DEV float stage_cvt(fft_half v, float*)
{
    return (float)v;
}
FFT_DEV fft_half stage_cvt(float v, fft_half*)
{
    return (fft_half)v;
}
FFT_DEV float2 stage_cvt(fft_half2 v, float2*)
{
    float2 r;
    r.x = (float)v.x;
    r.y = (float)v.y;
    return r;
}
FFT_DEV fft_half2 stage_cvt(float2 v, fft_half2*)
{
    fft_half2 r;
    r.x = (fft_half)v.x;
    r.y = (fft_half)v.y;
    return r;
}

// one element of a half-precision staging copy: U is the user's element type (half or half
// pair), E the scratch type (float or float pair)
template <typename U, typename E>
FFT_DEV void half_stage_elem(const fftk_cb_params& p, uint64_t gid)
{
    uint32_t i0 = (uint32_t)(gid % p.len[0]);
    gid /= p.len[0];
    uint32_t i1 = (uint32_t)(gid % p.len[1]);
    gid /= p.len[1];
    uint32_t i2 = (uint32_t)(gid % p.len[2]);
    uint64_t b  = gid / p.len[2];
    if(b >= p.batch)
        return;
    const size_t off = (size_t)(p.offset + (int64_t)b * p.dist + (int64_t)i0 * p.stride[0]
                                + (int64_t)i1 * p.stride[1] + (int64_t)i2 * p.stride[2]);
    U* user = static_cast<U*>(p.user);
    E* scr  = static_cast<E*>(p.scratch);
    if(!p.store)
        scr[off] = stage_cvt(user[off], static_cast<E*>(nullptr));
    else
        user[off] = stage_cvt(scr[off], static_cast<U*>(nullptr));
}

// one element of a callback copy (fftk_cb_params); E is the element type of the array
template <typename E>
FFT_DEV void callback_elem(const fftk_cb_params& p, uint64_t gid)
{
    typedef E (*load_fn)(E*, size_t, void*, void*);
    typedef void (*store_fn)(E*, size_t, E, void*, void*);
    uint32_t i0 = (uint32_t)(gid % p.len[0]);
    gid /= p.len[0];
    uint32_t i1 = (uint32_t)(gid % p.len[1]);
    gid /= p.len[1];
    uint32_t i2 = (uint32_t)(gid % p.len[2]);
    uint64_t b  = gid / p.len[2];
    if(b >= p.batch)
        return;
    const size_t off = (size_t)(p.offset + (int64_t)b * p.dist + (int64_t)i0 * p.stride[0]
                                + (int64_t)i1 * p.stride[1] + (int64_t)i2 * p.stride[2]);
    E* user = static_cast<E*>(p.user);
    E* scr  = static_cast<E*>(p.scratch);
    if(!p.store)
        scr[off] = p.fn ? reinterpret_cast<load_fn>(p.fn)(user, off, p.data, nullptr) : user[off];
    else if(p.fn)
        reinterpret_cast<store_fn>(p.fn)(user, off, scr[off], p.data, nullptr);
    else
        user[off] = scr[off];
}

// one element of a row copy (fftk_copy_params)
template <typename T>
FFT_DEV void copy_elem(const fftk_copy_params& p, uint64_t gid)
{
    uint32_t j  = (uint32_t)(gid % p.cnt);
    uint64_t r  = gid / p.cnt;
    uint32_t r0 = (uint32_t)(r % p.rows0);
    r /= p.rows0;
    uint32_t r1 = (uint32_t)(r % p.rows1);
    uint32_t r2 = (uint32_t)(r / p.rows1);
    if(r2 >= p.rows2)
        return;
    const int64_t sb   = (int64_t)r0 * p.s_r0 + (int64_t)r1 * p.s_r1 + (int64_t)r2 * p.s_r2;
    const int64_t db   = (int64_t)r0 * p.d_r0 + (int64_t)r1 * p.d_r1 + (int64_t)r2 * p.d_r2;
    const bool    flip = p.mirror_from && j >= p.mirror_from;
    const int64_t so   = sb + (int64_t)(flip ? p.mirror_n - j : j) * p.s_s;
    T             re, im;
    if(p.cb.load_fn)
    {
        if(p.src_real)
        {
            re = cb_load_scalar<T>(p.cb, so);
            im = 0;
        }
        else
        {
            typename cplx_of<T>::type v = cb_or_load<T>(p.cb, static_cast<const T*>(p.s0), static_cast<const T*>(p.s1), so);
            re                          = v.x;
            im                          = v.y;
        }
    }
    else
    {
        re = static_cast<const T*>(p.s0)[so];
        im = p.src_real ? (T)0 : static_cast<const T*>(p.s1)[so];
    }
    if(flip)
        im = -im;
    if(p.zero_im0 && j == 0)
        im = 0;
    if(p.use_scale)
    {
        re *= (T)p.scale;
        im *= (T)p.scale;
    }
    const int64_t dof           = db + (int64_t)j * p.d_s;
    if(p.cb.store_fn)
    {
        if(p.dst_real)
            cb_store_scalar<T>(p.cb, dof, re);
        else
        {
            typename cplx_of<T>::type v;
            v.x = re;
            v.y = im;
            cb_or_store<T>(p.cb, static_cast<T*>(p.d0), static_cast<T*>(p.d1), dof, v);
        }
        return;
    }
    static_cast<T*>(p.d0)[dof] = re;
    if(!p.dst_real)
        static_cast<T*>(p.d1)[dof] = im;
}

#endif
