/*
 * fft_oracle.c -- CPU restatement of the rocFFT transform path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the GPU library is
 * compared against; it is never linked into, loaded by or called from the
 * shipped library.  Only the test-suite, the smoke check and the benchmark's
 * CPU-baseline leg may use it.
 *
 * It restates, in plain C, the algorithms the reference executes on the GPU
 * (citations are paths under the reference tree, library/src unless noted):
 *   - in-LDS autosort Stockham passes with the stacked per-pass twiddle table
 *       device/generator/stockham_gen_base.h:347-456, twiddles.cpp:68-106,
 *       rtc_twiddle_gen.cpp:109-131
 *   - two-kernel large 1D (column FFT + multi-step large twiddle, row FFT with
 *     transposed store)
 *       tree_node_1D.cpp:404-469, device/generator/stockham_gen_cc.h:559-607,
 *       device/generator/rtc_radix_functions/large_twiddles.h:5-38,
 *       rtc_twiddle_gen.cpp:162-183
 *   - even-length real post-/pre-processing
 *       device/kernels/real2complex_device.h:25-103, :212-254
 *   - Bluestein chirp-z
 *       rtc_bluestein_gen.cpp:170-227, :324-380, rtc_chirp_gen.cpp:51-82,
 *       tree_node_bluestein.cpp:214-280
 *   - multi-dimensional real/complex composition and default contiguous layouts
 *       plan.cpp:87-197, tree_node_real.cpp:356-369, tree_node_2D.cpp:31-116
 *   - accuracy norms
 *       shared/accuracy_test.h:1497-1498, :1609-1619
 *
 * The reference's own CPU path is FFTW 3.3.9 (clients/tests/CMakeLists.txt:128-129),
 * which is a third-party dependency absent from the reference tree and from the
 * build image; parity is therefore anchored on the DFT definition
 * (orc_dft_naive_*), closed forms and library cross-checks held in the
 * test-suite.  Every function here is pinned by such a check; see
 * tests/test_oracle.py.
 *
 * Compiled twice: ORC_LD=0 -> double arithmetic (suffix _d), ORC_LD=1 -> long
 * double arithmetic (suffix _ld).  All external buffers are double.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#if ORC_LD
typedef long double real;
#define RCOS cosl
#define RSIN sinl
#define RSQRT sqrtl
#define RFABS fabsl
#define SUF(name) name##_ld
#define ORC_PI 3.141592653589793238462643383279502884L
#else
typedef double real;
#define RCOS cos
#define RSIN sin
#define RSQRT sqrt
#define RFABS fabs
#define SUF(name) name##_d
#define ORC_PI 3.141592653589793238462643383279502884
#endif

typedef struct
{
    real x, y;
} cplx;

static inline cplx cmul(cplx a, cplx b)
{
    cplx r = {a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x};
    return r;
}
static inline cplx cadd(cplx a, cplx b)
{
    cplx r = {a.x + b.x, a.y + b.y};
    return r;
}
static inline cplx csub(cplx a, cplx b)
{
    cplx r = {a.x - b.x, a.y - b.y};
    return r;
}

/* e^{sign * 2*pi*i * num/den}, num reduced exactly in integers first. */
static cplx unit_root(uint64_t num, uint64_t den, int sign)
{
    num %= den;
    /* octant reduction keeps the argument of cos/sin small */
    real a = (real)2 * ORC_PI * (real)num / (real)den;
    cplx r = {RCOS(a), (real)sign * RSIN(a)};
    return r;
}

/* ------------------------------------------------------------------------- */
/* DFT by definition: X_k = sum_n x_n e^{dir*2*pi*i*n*k/N}.  dir=-1 forward.
   (sign convention: plan.cpp:843-846, rtc_twiddle_gen.cpp:198).            */
void SUF(orc_dft_naive)(const double* in, double* out, size_t n, int dir)
{
    cplx* w = (cplx*)malloc(n * sizeof(cplx));
    for(size_t j = 0; j < n; ++j)
        w[j] = unit_root(j, n, dir);
    for(size_t k = 0; k < n; ++k)
    {
        real sx = 0, sy = 0, cx = 0, cy = 0; /* Kahan-compensated sums */
        for(size_t j = 0; j < n; ++j)
        {
            cplx t  = w[(uint64_t)j * k % n];
            real ax = (real)in[2 * j], ay = (real)in[2 * j + 1];
            real px = ax * t.x - ay * t.y - cx;
            real py = ax * t.y + ay * t.x - cy;
            real nx = sx + px, ny = sy + py;
            cx = (nx - sx) - px;
            cy = (ny - sy) - py;
            sx = nx;
            sy = ny;
        }
        out[2 * k]     = (double)sx;
        out[2 * k + 1] = (double)sy;
    }
    free(w);
}

/* One output bin of a length-n DFT, O(n); used for spot checks at sizes where
   the full naive DFT is too slow (e.g. n = 1000003).                       */
void SUF(orc_dft_bin)(const double* in, size_t n, size_t k, int dir, double* out2)
{
    real sx = 0, sy = 0, cx = 0, cy = 0;
    for(size_t j = 0; j < n; ++j)
    {
        uint64_t u  = (uint64_t)(((unsigned __int128)j * k) % n);
        cplx     t  = unit_root(u, n, dir);
        real     ax = (real)in[2 * j], ay = (real)in[2 * j + 1];
        real     px = ax * t.x - ay * t.y - cx;
        real     py = ax * t.y + ay * t.x - cy;
        real     nx = sx + px, ny = sy + py;
        cx = (nx - sx) - px;
        cy = (ny - sy) - py;
        sx = nx;
        sy = ny;
    }
    out2[0] = (double)sx;
    out2[1] = (double)sy;
}

/* ------------------------------------------------------------------------- */
/* Factorisation into the radices the kernel catalogue uses
   (device/kernel-generator.py:229-685 uses 2..17; pow2 prefers 16/8/4).     */
int SUF(orc_factorize)(size_t n, int* factors, int maxf)
{
    static const int pref[] = {16, 8, 4, 2, 3, 5, 7, 11, 13, 17};
    int              nf     = 0;
    size_t           m      = n;
    /* strip odd primes first so the power-of-two part is split greedily */
    for(int i = 4; i < 10; ++i)
        while(m % (size_t)pref[i] == 0 && m > 1)
        {
            if(nf >= maxf)
                return -1;
            factors[nf++] = pref[i];
            m /= (size_t)pref[i];
        }
    for(int i = 0; i < 4; ++i)
        while(m % (size_t)pref[i] == 0 && m > 1)
        {
            if(nf >= maxf)
                return -1;
            factors[nf++] = pref[i];
            m /= (size_t)pref[i];
        }
    if(m != 1)
        return 0; /* has a prime factor above 17: not Stockham-able */
    return nf;
}

/* Stacked twiddle table (twiddles.cpp:68-106, rtc_twiddle_gen.cpp:109-131):
   for pass p>=1 with radix w and cumulative height c = prod_{q<p} f_q the
   block at offset off_p holds T[off_p + j*(w-1) + k-1] = e^{-2 pi i jk/(c w)},
   j in [0,c), k in [1,w).  Returns the number of entries.                   */
static size_t stacked_twiddles(size_t n, const int* f, int nf, cplx* tbl)
{
    (void)n;
    size_t off = 0, c = 1;
    for(int p = 0; p < nf; ++p)
    {
        size_t w = (size_t)f[p];
        if(p > 0)
        {
            for(size_t j = 0; j < c; ++j)
                for(size_t k = 1; k < w; ++k)
                    if(tbl)
                        tbl[off + j * (w - 1) + k - 1] = unit_root(j * k, c * w, -1);
            off += c * (w - 1);
        }
        c *= w;
    }
    return off;
}

size_t SUF(orc_stacked_twiddles)(size_t n, const int* f, int nf, double* out)
{
    size_t cnt = stacked_twiddles(n, f, nf, NULL);
    if(out)
    {
        cplx* t = (cplx*)malloc((cnt + 1) * sizeof(cplx));
        stacked_twiddles(n, f, nf, t);
        for(size_t i = 0; i < cnt; ++i)
        {
            out[2 * i]     = (double)t[i].x;
            out[2 * i + 1] = (double)t[i].y;
        }
        free(t);
    }
    return cnt;
}

/* radix-w butterfly = DFT of size w by definition (the reference's FwdRadN /
   InvRadN in device/generator/rtc_radix_functions/ are factored forms of it). */
static void butterfly(cplx* r, int w, int dir)
{
    cplx tmp[32];
    for(int k = 0; k < w; ++k)
    {
        cplx s = {0, 0};
        for(int j = 0; j < w; ++j)
            s = cadd(s, cmul(r[j], unit_root((uint64_t)j * k, (uint64_t)w, dir)));
        tmp[k] = s;
    }
    memcpy(r, tmp, (size_t)w * sizeof(cplx));
}

/* Autosort Stockham (stockham_gen_base.h:347-456): pass p reads
   r_k = A[t + k*N/w], multiplies by the stacked twiddle for k>=1 when p>0
   (index c - f0 + (w-1)(t mod c) + k-1 in the reference, which equals
   off_p + (w-1)(t mod c) + k-1 with the offsets above), applies the radix-w
   butterfly and writes A'[(t div c)*w*c + (t mod c) + k*c].                 */
static void stockham(cplx* a, cplx* b, size_t n, const int* f, int nf, int dir)
{
    size_t cnt = stacked_twiddles(n, f, nf, NULL);
    cplx*  tw  = (cplx*)malloc((cnt + 1) * sizeof(cplx));
    stacked_twiddles(n, f, nf, tw);
    size_t c = 1, off = 0;
    cplx * src = a, *dst = b;
    for(int p = 0; p < nf; ++p)
    {
        int    w = f[p];
        size_t m = n / (size_t)w;
        for(size_t t = 0; t < m; ++t)
        {
            cplx r[32];
            for(int k = 0; k < w; ++k)
                r[k] = src[t + (size_t)k * m];
            if(p > 0)
                for(int k = 1; k < w; ++k)
                {
                    cplx tv = tw[off + (size_t)(w - 1) * (t % c) + (size_t)k - 1];
                    if(dir > 0)
                        tv.y = -tv.y;
                    r[k] = cmul(r[k], tv);
                }
            butterfly(r, w, dir);
            for(int k = 0; k < w; ++k)
                dst[(t / c) * (size_t)w * c + (t % c) + (size_t)k * c] = r[k];
        }
        if(p > 0)
            off += c * (size_t)(w - 1);
        c *= (size_t)w;
        cplx* s = src;
        src     = dst;
        dst     = s;
    }
    if(src != a)
        memcpy(a, src, n * sizeof(cplx));
    free(tw);
}

void SUF(orc_stockham)(double* data, size_t n, const int* f, int nf, int dir)
{
    cplx* a = (cplx*)malloc(2 * n * sizeof(cplx));
    for(size_t i = 0; i < n; ++i)
    {
        a[i].x = (real)data[2 * i];
        a[i].y = (real)data[2 * i + 1];
    }
    stockham(a, a + n, n, f, nf, dir);
    for(size_t i = 0; i < n; ++i)
    {
        data[2 * i]     = (double)a[i].x;
        data[2 * i + 1] = (double)a[i].y;
    }
    free(a);
}

/* ------------------------------------------------------------------------- */
/* Fast production-shaped radix-2/4 kernel for powers of two, used inside the
   Bluestein convolution and for the long power-of-two lengths so that the
   oracle finishes in seconds; validated against stockham()/naive in tests.  */
static void fft_pow2(cplx* a, size_t n, int dir, const cplx* w /* n/2 roots, forward */)
{
    /* bit reversal */
    for(size_t i = 1, j = 0; i < n; ++i)
    {
        size_t bit = n >> 1;
        for(; j & bit; bit >>= 1)
            j ^= bit;
        j ^= bit;
        if(i < j)
        {
            cplx t = a[i];
            a[i]   = a[j];
            a[j]   = t;
        }
    }
    for(size_t len = 2; len <= n; len <<= 1)
    {
        size_t half = len >> 1, step = n / len;
        for(size_t i = 0; i < n; i += len)
            for(size_t k = 0; k < half; ++k)
            {
                cplx t = w[k * step];
                if(dir > 0)
                    t.y = -t.y;
                cplx u = a[i + k], v = cmul(a[i + k + half], t);
                a[i + k]        = cadd(u, v);
                a[i + k + half] = csub(u, v);
            }
    }
}

typedef struct
{
    size_t n;
    int    kind; /* 0 = trivial, 1 = pow2, 2 = stockham mixed radix, 3 = bluestein */
    int    f[64];
    int    nf;
    cplx*  w;     /* pow2: n/2 forward roots */
    size_t m;     /* bluestein padded length */
    cplx*  wm;    /* bluestein: m/2 forward roots */
    cplx*  chirp; /* bluestein: c_n = e^{+i pi n^2/N}, n<N (forward-transform chirp) */
} plan1d;

static size_t next_pow2(size_t v)
{
    size_t p = 1;
    while(p < v)
        p <<= 1;
    return p;
}

static plan1d* plan1d_create(size_t n)
{
    plan1d* p = (plan1d*)calloc(1, sizeof(plan1d));
    p->n      = n;
    if(n <= 1)
    {
        p->kind = 0;
        return p;
    }
    if((n & (n - 1)) == 0)
    {
        p->kind = 1;
        p->w    = (cplx*)malloc((n / 2 + 1) * sizeof(cplx));
        for(size_t j = 0; j < n / 2; ++j)
            p->w[j] = unit_root(j, n, -1);
        return p;
    }
    p->nf = SUF(orc_factorize)(n, p->f, 64);
    if(p->nf > 0)
    {
        p->kind = 2;
        return p;
    }
    /* Bluestein (tree_node_bluestein.cpp:27-61 picks the padded length; any
       M >= 2N-1 gives the same mathematical result, a power of two is used). */
    p->kind = 3;
    p->m    = next_pow2(2 * n - 1);
    p->wm   = (cplx*)malloc((p->m / 2 + 1) * sizeof(cplx));
    for(size_t j = 0; j < p->m / 2; ++j)
        p->wm[j] = unit_root(j, p->m, -1);
    p->chirp = (cplx*)malloc(n * sizeof(cplx));
    for(size_t j = 0; j < n; ++j)
    {
        /* exact n^2 mod 2N (rtc_chirp_gen.cpp:51-82 does the same reduction
           with 32-bit halves); angle = pi * (j^2 mod 2N) / N                */
        uint64_t u  = (uint64_t)(((unsigned __int128)j * j) % (2 * (uint64_t)n));
        p->chirp[j] = unit_root(u, 2 * (uint64_t)n, +1);
    }
    return p;
}

static void plan1d_destroy(plan1d* p)
{
    if(!p)
        return;
    free(p->w);
    free(p->wm);
    free(p->chirp);
    free(p);
}

/* Bluestein, rtc_bluestein_gen.cpp:170-227 (chirp layout with wrap-around),
   :324-346 (pad_mul: a_n = x_n * conj(c_n), zero padded), :348-359 (fft_mul),
   :361-380 (res_mul: X_k = (1/M) y_k conj(c_k)); for the forward transform
   c_n = e^{+i pi n^2/N}, the inverse transform uses the conjugate chirp.     */
static void bluestein(const plan1d* p, cplx* x, int dir, cplx* work /* 2*m */)
{
    size_t n = p->n, m = p->m;
    cplx * a = work, *b = work + m;
    for(size_t j = 0; j < m; ++j)
    {
        a[j].x = a[j].y = 0;
        b[j].x = b[j].y = 0;
    }
    for(size_t j = 0; j < n; ++j)
    {
        cplx c = p->chirp[j];
        if(dir > 0)
            c.y = -c.y; /* inverse transform: conjugate chirp */
        cplx cc = {c.x, -c.y};
        a[j]    = cmul(x[j], cc);
        b[j]    = c;
        if(j)
            b[m - j] = c;
    }
    fft_pow2(a, m, -1, p->wm);
    fft_pow2(b, m, -1, p->wm);
    for(size_t j = 0; j < m; ++j)
        a[j] = cmul(a[j], b[j]);
    fft_pow2(a, m, +1, p->wm);
    real mi = (real)1 / (real)m;
    for(size_t k = 0; k < n; ++k)
    {
        cplx c = p->chirp[k];
        if(dir > 0)
            c.y = -c.y;
        cplx cc = {c.x, -c.y};
        cplx r  = cmul(a[k], cc);
        x[k].x  = r.x * mi;
        x[k].y  = r.y * mi;
    }
}

static void plan1d_exec(const plan1d* p, cplx* x, int dir, cplx* work)
{
    switch(p->kind)
    {
    case 0:
        return;
    case 1:
        fft_pow2(x, p->n, dir, p->w);
        return;
    case 2:
        stockham(x, work, p->n, p->f, p->nf, dir);
        return;
    default:
        bluestein(p, x, dir, work);
        return;
    }
}

static size_t plan1d_worksize(const plan1d* p)
{
    if(p->kind == 3)
        return 2 * p->m;
    return p->n + 1;
}

/* Batched contiguous 1D complex transform, any n (test entry point).        */
void SUF(orc_fft1d)(double* data, size_t n, size_t batch, int dir)
{
    plan1d* p = plan1d_create(n);
#pragma omp parallel
    {
        cplx* x    = (cplx*)malloc(n * sizeof(cplx));
        cplx* work = (cplx*)malloc(plan1d_worksize(p) * sizeof(cplx));
#pragma omp for schedule(static)
        for(long b = 0; b < (long)batch; ++b)
        {
            double* d = data + 2 * n * (size_t)b;
            for(size_t i = 0; i < n; ++i)
            {
                x[i].x = (real)d[2 * i];
                x[i].y = (real)d[2 * i + 1];
            }
            plan1d_exec(p, x, dir, work);
            for(size_t i = 0; i < n; ++i)
            {
                d[2 * i]     = (double)x[i].x;
                d[2 * i + 1] = (double)x[i].y;
            }
        }
        free(x);
        free(work);
    }
    plan1d_destroy(p);
}

/* Bluestein forced for any n (so the chirp-z restatement can be checked on
   lengths that would otherwise take the Stockham route).                    */
void SUF(orc_bluestein1d)(double* data, size_t n, int dir)
{
    plan1d* p = (plan1d*)calloc(1, sizeof(plan1d));
    p->n      = n;
    p->kind   = 3;
    p->m      = next_pow2(2 * n - 1);
    p->wm     = (cplx*)malloc((p->m / 2 + 1) * sizeof(cplx));
    for(size_t j = 0; j < p->m / 2; ++j)
        p->wm[j] = unit_root(j, p->m, -1);
    p->chirp = (cplx*)malloc(n * sizeof(cplx));
    for(size_t j = 0; j < n; ++j)
    {
        uint64_t u  = (uint64_t)(((unsigned __int128)j * j) % (2 * (uint64_t)n));
        p->chirp[j] = unit_root(u, 2 * (uint64_t)n, +1);
    }
    cplx* x    = (cplx*)malloc(n * sizeof(cplx));
    cplx* work = (cplx*)malloc(2 * p->m * sizeof(cplx));
    for(size_t i = 0; i < n; ++i)
    {
        x[i].x = (real)data[2 * i];
        x[i].y = (real)data[2 * i + 1];
    }
    bluestein(p, x, dir, work);
    for(size_t i = 0; i < n; ++i)
    {
        data[2 * i]     = (double)x[i].x;
        data[2 * i + 1] = (double)x[i].y;
    }
    free(x);
    free(work);
    plan1d_destroy(p);
}

/* ------------------------------------------------------------------------- */
/* Large-1D twiddle W_L^u as a product of table rows
   (large_twiddles.h:5-38, rtc_twiddle_gen.cpp:162-183):
   Tbl[s*2^base + j] = e^{-2 pi i j 2^{s base}/L};
   W_L^u = prod_s Tbl[s*2^base + ((u >> s*base) & (2^base-1))].              */
static cplx large_twiddle(const cplx* tbl, int base, int steps, uint64_t u)
{
    cplx   r    = tbl[u & ((1u << base) - 1)];
    size_t rows = (size_t)1 << base;
    for(int s = 1; s < steps; ++s)
        r = cmul(r, tbl[(size_t)s * rows + ((u >> (s * base)) & ((1u << base) - 1))]);
    return r;
}

void SUF(orc_large_twiddle)(size_t L, int base, int steps, uint64_t u, double* out2)
{
    size_t rows = (size_t)1 << base;
    cplx*  tbl  = (cplx*)malloc(rows * (size_t)steps * sizeof(cplx));
    for(int s = 0; s < steps; ++s)
        for(size_t j = 0; j < rows; ++j)
        {
            /* j * 2^{s base} may exceed L: reduce exactly */
            unsigned __int128 e = (unsigned __int128)j << (s * base);
            tbl[(size_t)s * rows + j] = unit_root((uint64_t)(e % L), L, -1);
        }
    cplx r  = large_twiddle(tbl, base, steps, u);
    out2[0] = (double)r.x;
    out2[1] = (double)r.y;
    free(tbl);
}

/* Two-kernel large 1D (tree_node_1D.cpp:404-469): L = N1*N0, n = n1*N0 + n0.
   Kernel A: for every n0 an N1-point FFT over n1, result k1 multiplied by
   W_L^{k1*n0}, stored at k1*N0 + n0.  Kernel B: for every k1 an N0-point FFT
   over n0, stored transposed at k0*N1 + k1.                                  */
void SUF(orc_large1d_cc)(double* data, size_t n1, size_t n0, int base, int steps, int dir)
{
    size_t L    = n1 * n0;
    size_t rows = (size_t)1 << base;
    cplx*  tbl  = (cplx*)malloc(rows * (size_t)steps * sizeof(cplx));
    for(int s = 0; s < steps; ++s)
        for(size_t j = 0; j < rows; ++j)
        {
            unsigned __int128 e = (unsigned __int128)j << (s * base);
            tbl[(size_t)s * rows + j] = unit_root((uint64_t)(e % L), L, -1);
        }
    cplx* a = (cplx*)malloc(L * sizeof(cplx));
    cplx* b = (cplx*)malloc(L * sizeof(cplx));
    for(size_t i = 0; i < L; ++i)
    {
        a[i].x = (real)data[2 * i];
        a[i].y = (real)data[2 * i + 1];
    }
    plan1d* p1   = plan1d_create(n1);
    plan1d* p0   = plan1d_create(n0);
    size_t  wmax = plan1d_worksize(p1) > plan1d_worksize(p0) ? plan1d_worksize(p1)
                                                              : plan1d_worksize(p0);
    cplx*   work = (cplx*)malloc(wmax * sizeof(cplx));
    cplx*   line = (cplx*)malloc((n1 > n0 ? n1 : n0) * sizeof(cplx));
    for(size_t c0 = 0; c0 < n0; ++c0)
    {
        for(size_t j = 0; j < n1; ++j)
            line[j] = a[j * n0 + c0];
        plan1d_exec(p1, line, dir, work);
        for(size_t k1 = 0; k1 < n1; ++k1)
        {
            cplx t = large_twiddle(tbl, base, steps, (uint64_t)k1 * c0);
            if(dir > 0)
                t.y = -t.y;
            b[k1 * n0 + c0] = cmul(line[k1], t);
        }
    }
    for(size_t k1 = 0; k1 < n1; ++k1)
    {
        for(size_t j = 0; j < n0; ++j)
            line[j] = b[k1 * n0 + j];
        plan1d_exec(p0, line, dir, work);
        for(size_t k0 = 0; k0 < n0; ++k0)
            a[k0 * n1 + k1] = line[k0];
    }
    for(size_t i = 0; i < L; ++i)
    {
        data[2 * i]     = (double)a[i].x;
        data[2 * i + 1] = (double)a[i].y;
    }
    free(a);
    free(b);
    free(work);
    free(line);
    free(tbl);
    plan1d_destroy(p1);
    plan1d_destroy(p0);
}

/* ------------------------------------------------------------------------- */
/* Even-length real transforms (real2complex_device.h:25-103 and :212-254).
   z holds the half-length complex FFT Z of the packed reals; writes the
   half+1 Hermitian bins.  T_k = e^{-2 pi i k/N}, N = 2*half.                 */
static void r2c_post(const cplx* z, cplx* out, size_t half)
{
    out[0].x    = z[0].x + z[0].y;
    out[0].y    = 0;
    out[half].x = z[0].x - z[0].y;
    out[half].y = 0;
    for(size_t p = 1; p <= half / 2; ++p)
    {
        size_t q = half - p;
        if(p == q)
        {
            out[p].x = z[p].x;
            out[p].y = -z[p].y;
            continue;
        }
        cplx zp = z[p], zq = z[q];
        cplx u  = {(real)0.5 * (zp.x + zq.x), (real)0.5 * (zp.y + zq.y)};
        cplx v  = {(real)0.5 * (zp.x - zq.x), (real)0.5 * (zp.y - zq.y)};
        cplx t  = unit_root(p, 2 * half, -1);
        out[p].x = u.x + v.x * t.y + u.y * t.x;
        out[p].y = v.y + u.y * t.y - v.x * t.x;
        out[q].x = u.x - v.x * t.y - u.y * t.x;
        out[q].y = -v.y + u.y * t.y - v.x * t.x;
    }
}

/* Inverse pre-processing: Hermitian bins -> half-length complex input of the
   inverse FFT (unnormalised, the factor 2 is built in).  Uses only the real
   parts of bins 0 and N/2 (real2complex_device.h:226-231).                   */
static void c2r_pre(const cplx* in, cplx* z, size_t half)
{
    z[0].x = in[0].x + in[half].x;
    z[0].y = in[0].x - in[half].x;
    for(size_t p = 1; p <= half / 2; ++p)
    {
        size_t q = half - p;
        if(p == q)
        {
            z[p].x = (real)2 * in[p].x;
            z[p].y = (real)-2 * in[p].y;
            continue;
        }
        cplx a = in[p], b = in[q];
        cplx u = cadd(a, b), v = csub(a, b);
        cplx t = unit_root(p, 2 * half, -1);
        z[p].x = u.x + v.x * t.y - u.y * t.x;
        z[p].y = v.y + u.y * t.y + v.x * t.x;
        z[q].x = u.x - v.x * t.y + u.y * t.x;
        z[q].y = -v.y + u.y * t.y + v.x * t.x;
    }
}

void SUF(orc_r2c_post)(const double* z, double* out, size_t half)
{
    cplx* a = (cplx*)malloc(half * sizeof(cplx));
    cplx* o = (cplx*)malloc((half + 1) * sizeof(cplx));
    for(size_t i = 0; i < half; ++i)
    {
        a[i].x = (real)z[2 * i];
        a[i].y = (real)z[2 * i + 1];
    }
    r2c_post(a, o, half);
    for(size_t i = 0; i <= half; ++i)
    {
        out[2 * i]     = (double)o[i].x;
        out[2 * i + 1] = (double)o[i].y;
    }
    free(a);
    free(o);
}

void SUF(orc_c2r_pre)(const double* in, double* z, size_t half)
{
    cplx* a = (cplx*)malloc((half + 1) * sizeof(cplx));
    cplx* o = (cplx*)malloc(half * sizeof(cplx));
    for(size_t i = 0; i <= half; ++i)
    {
        a[i].x = (real)in[2 * i];
        a[i].y = (real)in[2 * i + 1];
    }
    c2r_pre(a, o, half);
    for(size_t i = 0; i < half; ++i)
    {
        z[2 * i]     = (double)o[i].x;
        z[2 * i + 1] = (double)o[i].y;
    }
    free(a);
    free(o);
}

/* ------------------------------------------------------------------------- */
/* Whole transforms at the API's default contiguous layout (plan.cpp:87-197):
   lengths[0] is the fastest dimension; real forward output has
   lengths[0]/2+1 bins along dimension 0; batches are back to back.
   type: 0 complex forward, 1 complex inverse, 2 real forward, 3 real inverse
   (rocfft.h:91-97).  Unnormalised in both directions.                        */

/* strided in-place 1D pass over a complex array */
static void pass_dim(cplx*         a,
                     const plan1d* p,
                     size_t        n,
                     size_t        stride,
                     size_t        count_lo,
                     size_t        count_hi,
                     size_t        stride_hi,
                     int           dir)
{
    /* lines: for hi in [0,count_hi), lo in [0,count_lo): base = hi*stride_hi + lo */
    long total = (long)(count_lo * count_hi);
#pragma omp parallel
    {
        cplx* line = (cplx*)malloc(n * sizeof(cplx));
        cplx* work = (cplx*)malloc(plan1d_worksize(p) * sizeof(cplx));
#pragma omp for schedule(static)
        for(long l = 0; l < total; ++l)
        {
            size_t lo = (size_t)l % count_lo, hi = (size_t)l / count_lo;
            cplx*  base = a + hi * stride_hi + lo;
            if(stride == 1)
                plan1d_exec(p, base, dir, work);
            else
            {
                for(size_t j = 0; j < n; ++j)
                    line[j] = base[j * stride];
                plan1d_exec(p, line, dir, work);
                for(size_t j = 0; j < n; ++j)
                    base[j * stride] = line[j];
            }
        }
        free(line);
        free(work);
    }
}

static void complex_nd(cplx* a, size_t rank, const size_t* len, size_t batch, int dir)
{
    size_t total = 1;
    for(size_t d = 0; d < rank; ++d)
        total *= len[d];
    size_t stride = 1;
    for(size_t d = 0; d < rank; ++d)
    {
        plan1d* p = plan1d_create(len[d]);
        /* lines along d: lo = indices below d (count = stride), hi = the rest */
        size_t count_hi = total / (stride * len[d]) * batch;
        pass_dim(a, p, len[d], stride, stride, count_hi, stride * len[d], dir);
        plan1d_destroy(p);
        stride *= len[d];
    }
}

int SUF(orc_transform)(int           type,
                       size_t        rank,
                       const size_t* len,
                       size_t        batch,
                       const double* in,
                       double*       out)
{
    if(rank < 1 || rank > 3)
        return 1;
    size_t total = 1;
    for(size_t d = 0; d < rank; ++d)
        total *= len[d];
    if(type == 0 || type == 1)
    {
        int   dir = type == 0 ? -1 : +1;
        cplx* a   = (cplx*)malloc(total * batch * sizeof(cplx));
        for(size_t i = 0; i < total * batch; ++i)
        {
            a[i].x = (real)in[2 * i];
            a[i].y = (real)in[2 * i + 1];
        }
        complex_nd(a, rank, len, batch, dir);
        for(size_t i = 0; i < total * batch; ++i)
        {
            out[2 * i]     = (double)a[i].x;
            out[2 * i + 1] = (double)a[i].y;
        }
        free(a);
        return 0;
    }
    size_t n0    = len[0];
    size_t h0    = n0 / 2 + 1;
    size_t rows  = total / n0 * batch; /* number of dimension-0 lines */
    cplx*  hb    = (cplx*)malloc(rows * h0 * sizeof(cplx));
    if(type == 2)
    {
        /* dimension 0: real -> Hermitian */
        if(n0 % 2 == 0)
        {
            /* tree_node_real.cpp:356-369: view the reals as n0/2 complexes */
            size_t  half = n0 / 2;
            plan1d* p    = plan1d_create(half);
#pragma omp parallel
            {
                cplx* z    = (cplx*)malloc((half + 1) * sizeof(cplx));
                cplx* work = (cplx*)malloc(plan1d_worksize(p) * sizeof(cplx));
#pragma omp for schedule(static)
                for(long r = 0; r < (long)rows; ++r)
                {
                    const double* x = in + (size_t)r * n0;
                    for(size_t j = 0; j < half; ++j)
                    {
                        z[j].x = (real)x[2 * j];
                        z[j].y = (real)x[2 * j + 1];
                    }
                    plan1d_exec(p, z, -1, work);
                    r2c_post(z, hb + (size_t)r * h0, half);
                }
                free(z);
                free(work);
            }
            plan1d_destroy(p);
        }
        else
        {
            /* odd length: embed as complex, full transform, keep h0 bins
               (tree_node_real.cpp:115-206)                                  */
            plan1d* p = plan1d_create(n0);
#pragma omp parallel
            {
                cplx* z    = (cplx*)malloc(n0 * sizeof(cplx));
                cplx* work = (cplx*)malloc(plan1d_worksize(p) * sizeof(cplx));
#pragma omp for schedule(static)
                for(long r = 0; r < (long)rows; ++r)
                {
                    const double* x = in + (size_t)r * n0;
                    for(size_t j = 0; j < n0; ++j)
                    {
                        z[j].x = (real)x[j];
                        z[j].y = 0;
                    }
                    plan1d_exec(p, z, -1, work);
                    memcpy(hb + (size_t)r * h0, z, h0 * sizeof(cplx));
                }
                free(z);
                free(work);
            }
            plan1d_destroy(p);
        }
        /* remaining dimensions: complex forward on the Hermitian array */
        size_t stride = h0;
        size_t htotal = total / n0 * h0;
        for(size_t d = 1; d < rank; ++d)
        {
            plan1d* p        = plan1d_create(len[d]);
            size_t  count_hi = htotal / (stride * len[d]) * batch;
            pass_dim(hb, p, len[d], stride, stride, count_hi, stride * len[d], -1);
            plan1d_destroy(p);
            stride *= len[d];
        }
        for(size_t i = 0; i < rows * h0; ++i)
        {
            out[2 * i]     = (double)hb[i].x;
            out[2 * i + 1] = (double)hb[i].y;
        }
        free(hb);
        return 0;
    }
    if(type == 3)
    {
        for(size_t i = 0; i < rows * h0; ++i)
        {
            hb[i].x = (real)in[2 * i];
            hb[i].y = (real)in[2 * i + 1];
        }
        /* higher dimensions first (tree_node_real.cpp:1573-1651 order), then
           dimension 0 complex -> real                                        */
        size_t stride = h0;
        size_t htotal = total / n0 * h0;
        for(size_t d = 1; d < rank; ++d)
        {
            plan1d* p        = plan1d_create(len[d]);
            size_t  count_hi = htotal / (stride * len[d]) * batch;
            pass_dim(hb, p, len[d], stride, stride, count_hi, stride * len[d], +1);
            plan1d_destroy(p);
            stride *= len[d];
        }
        if(n0 % 2 == 0)
        {
            size_t  half = n0 / 2;
            plan1d* p    = plan1d_create(half);
#pragma omp parallel
            {
                cplx* z    = (cplx*)malloc((half + 1) * sizeof(cplx));
                cplx* work = (cplx*)malloc(plan1d_worksize(p) * sizeof(cplx));
#pragma omp for schedule(static)
                for(long r = 0; r < (long)rows; ++r)
                {
                    c2r_pre(hb + (size_t)r * h0, z, half);
                    plan1d_exec(p, z, +1, work);
                    double* x = out + (size_t)r * n0;
                    for(size_t j = 0; j < half; ++j)
                    {
                        x[2 * j]     = (double)z[j].x;
                        x[2 * j + 1] = (double)z[j].y;
                    }
                }
                free(z);
                free(work);
            }
            plan1d_destroy(p);
        }
        else
        {
            plan1d* p = plan1d_create(n0);
#pragma omp parallel
            {
                cplx* z    = (cplx*)malloc(n0 * sizeof(cplx));
                cplx* work = (cplx*)malloc(plan1d_worksize(p) * sizeof(cplx));
#pragma omp for schedule(static)
                for(long r = 0; r < (long)rows; ++r)
                {
                    const cplx* h = hb + (size_t)r * h0;
                    /* expand the Hermitian half (imaginary part of bin 0 ignored) */
                    z[0].x = h[0].x;
                    z[0].y = 0;
                    for(size_t k = 1; k < h0; ++k)
                    {
                        z[k]        = h[k];
                        z[n0 - k].x = h[k].x;
                        z[n0 - k].y = -h[k].y;
                    }
                    plan1d_exec(p, z, +1, work);
                    double* x = out + (size_t)r * n0;
                    for(size_t j = 0; j < n0; ++j)
                        x[j] = (double)z[j].x;
                }
                free(z);
                free(work);
            }
            plan1d_destroy(p);
        }
        free(hb);
        return 0;
    }
    free(hb);
    return 1;
}

/* ------------------------------------------------------------------------- */
/* Norms (shared/accuracy_test.h:1497-1498, :1609-1619; shared/fft_params.h
   :2657-2745): returns relative L2 = ||a-b||_2/||b||_2 and relative
   Linf = ||a-b||_inf/||b||_inf over `count` doubles.                         */
void SUF(orc_rel_norms)(const double* a, const double* b, size_t count, double* l2, double* linf)
{
    real s2 = 0, r2 = 0, si = 0, ri = 0;
    for(size_t i = 0; i < count; ++i)
    {
        real d = (real)a[i] - (real)b[i];
        s2 += d * d;
        r2 += (real)b[i] * (real)b[i];
        if(RFABS(d) > si)
            si = RFABS(d);
        if(RFABS((real)b[i]) > ri)
            ri = RFABS((real)b[i]);
    }
    *l2   = r2 > 0 ? (double)RSQRT(s2 / r2) : (double)RSQRT(s2);
    *linf = ri > 0 ? (double)(si / ri) : (double)si;
}

int SUF(orc_num_threads)(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
