// plan.cpp -- planner, table builders and executor (host only, no HIP types).
#include "plan.h"
#include "gpu_rt.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <thread>

namespace fftamd
{

// ---------------------------------------------------------------------------
// limits of the tile kernel on gfx950

static const size_t   LDS_SOFT_BYTES = 64 * 1024;  // preferred tile footprint (two workgroups per CU)
static const size_t   LDS_HARD_BYTES = 160 * 1024; // LDS of one CU
static const size_t   LDS_COL_BYTES  = 80 * 1024;  // a column tile may grow to this to keep its rows wide
static const size_t   LDS_WIDE_BYTES = 140 * 1024; // ... and to this when the alternative is a second pass
static const uint32_t MAX_THREADS    = 512;
// a few compiled kernels for long single-precision rows use one workgroup of up to this many threads
static const uint32_t WIDE_THREADS   = 1024;
static const uint32_t PADSHIFT       = 4;
// a strided ("column") pass wants at least this many bytes contiguous per row of its tile
static const size_t   COL_RUN_BYTES  = 128;

// ROCFFT_AMD_GENERIC=1 forces the generic tile kernel everywhere (A/B comparisons)
static const bool g_use_fast_env = !getenv("ROCFFT_AMD_GENERIC");
// set while the alternate plan for buffers without vector alignment is being built: only the
// run-time-schedule tile kernel, which has a scalar-access form for every pass
static thread_local bool t_generic_only = false;
static bool use_fast_kernels()
{
    return g_use_fast_env && !t_generic_only;
}
#define g_use_fast use_fast_kernels()
// ROCFFT_AMD_NO_XCD_REMAP=1 keeps the hardware's round-robin workgroup order (A/B comparisons)
static const bool g_xcd_remap = !getenv("ROCFFT_AMD_NO_XCD_REMAP");
static const bool g_share_first = !getenv("ROCFFT_AMD_NO_SHARE_FIRST");
static const bool g_fold_tiles = !getenv("ROCFFT_AMD_NO_FOLD");

struct PlanError : std::runtime_error
{
    rocfft_status status;
    PlanError(rocfft_status s, const std::string& what)
        : std::runtime_error(what)
        , status(s)
    {
    }
};

static void fail(const std::string& what)
{
    throw PlanError(rocfft_status_failure, what);
}

// ---------------------------------------------------------------------------
// tables (computed in long double on the host, narrowed to the plan precision;
// the reference computes its tables in double on the device:
// library/src/rtc_twiddle_gen.cpp:103-188, library/src/rtc_chirp_gen.cpp:51-82)

DeviceTable::~DeviceTable()
{
    if(dptr)
        fftrt_free(dptr);
}

static const long double PI_L = 3.141592653589793238462643383279502884L;

static void unit_root(uint64_t num, uint64_t den, long double& c, long double& s)
{
    // e^{-2 pi i num/den}; reduce to the first octant so cos/sin see small arguments
    num %= den;
    // exact symmetries keep tables bit-symmetric: handle multiples of den/8 exactly
    long double a = 2.0L * PI_L * (long double)num / (long double)den;
    c             = cosl(a);
    s             = -sinl(a);
    if(num == 0)
    {
        c = 1;
        s = 0;
    }
    else if(4 * num == den)
    {
        c = 0;
        s = -1;
    }
    else if(2 * num == den)
    {
        c = -1;
        s = 0;
    }
    else if(4 * num == 3 * den)
    {
        c = 0;
        s = 1;
    }
}

struct HostTable
{
    std::vector<long double> v; // (re, im) pairs
    void                     push(long double c, long double s)
    {
        v.push_back(c);
        v.push_back(s);
    }
};

// fn(first, last) over [0, n) on the host's threads (long tables: the chirp of a prime length in
// the millions costs seconds on one thread)
template <typename Fn>
static void host_parallel(uint64_t n, Fn fn)
{
    unsigned workers = std::min<unsigned>(16, std::max(1u, std::thread::hardware_concurrency()));
    if(n < (1u << 16) || workers < 2)
    {
        fn((uint64_t)0, n);
        return;
    }
    std::vector<std::thread> pool;
    const uint64_t           step = (n + workers - 1) / workers;
    for(unsigned w = 0; w < workers; ++w)
    {
        const uint64_t a = std::min<uint64_t>(n, w * step), b = std::min<uint64_t>(n, a + step);
        if(a < b)
            pool.emplace_back([=]() { fn(a, b); });
    }
    for(std::thread& t : pool)
        t.join();
}

static std::mutex                                   g_cache_mutex;
static std::map<std::string, std::weak_ptr<DeviceTable>> g_cache;

void table_cache_clear()
{
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    for(auto it = g_cache.begin(); it != g_cache.end();)
    {
        if(it->second.expired())
            it = g_cache.erase(it);
        else
            ++it;
    }
}

static TablePtr upload_table(const HostTable& h, int precision, bool dry)
{
    TablePtr t(new DeviceTable);
    size_t   count = h.v.size();
    t->bytes       = count * (precision ? sizeof(double) : sizeof(float));
    if(dry || count == 0)
        return t;
    if(fftrt_malloc(&t->dptr, t->bytes) != 0)
        fail("device allocation of a table failed");
    int rc;
    if(precision)
    {
        std::vector<double> d(count);
        for(size_t i = 0; i < count; ++i)
            d[i] = (double)h.v[i];
        rc = fftrt_upload(t->dptr, d.data(), t->bytes);
    }
    else
    {
        std::vector<float> d(count);
        for(size_t i = 0; i < count; ++i)
            d[i] = (float)h.v[i];
        rc = fftrt_upload(t->dptr, d.data(), t->bytes);
    }
    if(rc != 0)
        fail("upload of a table failed");
    return t;
}

template <typename Gen>
static TablePtr cached_table(const std::string& key, int precision, bool dry, Gen gen)
{
    int dev = 0;
    if(!dry)
        fftrt_device_info(&dev, nullptr, nullptr, nullptr, 0);
    std::ostringstream k;
    k << key << "/p" << precision << "/d" << dev << (dry ? "/dry" : "");
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto                        it = g_cache.find(k.str());
    if(it != g_cache.end())
        if(TablePtr t = it->second.lock())
            return t;
    HostTable h;
    if(!dry) // a plan that is only described needs no table contents
        gen(h);
    TablePtr t       = upload_table(h, precision, dry);
    g_cache[k.str()] = t;
    return t;
}

// stacked per-pass twiddles: pass p (radix w, cumulative height c) holds
// e^{-2 pi i jk/(c w)} at off_p + (k-1)*c + j
static TablePtr stacked_twiddles(const std::vector<uint32_t>& radix, int precision, bool dry,
                                 uint32_t* twoff)
{
    std::ostringstream key;
    key << "stk";
    for(uint32_t r : radix)
        key << "_" << r;
    uint32_t off = 0, c = 1;
    for(size_t p = 0; p < radix.size(); ++p)
    {
        twoff[p] = off;
        if(p > 0)
            off += c * (radix[p] - 1);
        c *= radix[p];
    }
    return cached_table(key.str(), precision, dry, [&](HostTable& h) {
        uint32_t cc = 1;
        for(size_t p = 0; p < radix.size(); ++p)
        {
            uint32_t w = radix[p];
            if(p > 0)
                for(uint32_t k = 1; k < w; ++k)
                    for(uint32_t j = 0; j < cc; ++j)
                    {
                        long double co, si;
                        unit_root((uint64_t)j * k, (uint64_t)cc * w, co, si);
                        h.push(co, si);
                    }
            cc *= w;
        }
        if(h.v.empty())
            h.push(1, 0);
    });
}

// two-level table for W_L^u = lo[u & mask] * hi[u >> shift]
static uint32_t large_twiddle_shift(uint64_t L)
{
    uint32_t bits = 0;
    while(((uint64_t)1 << bits) < L)
        ++bits;
    return (bits + 1) / 2;
}

static TablePtr large_twiddles(uint64_t L, int precision, bool dry)
{
    std::ostringstream key;
    key << "ltw_" << L;
    return cached_table(key.str(), precision, dry, [&](HostTable& h) {
        uint32_t shift = large_twiddle_shift(L);
        uint64_t lo    = (uint64_t)1 << shift;
        uint64_t hi    = (L + lo - 1) / lo + 1;
        for(uint64_t j = 0; j < lo; ++j)
        {
            long double c, s;
            unit_root(j, L, c, s);
            h.push(c, s);
        }
        for(uint64_t j = 0; j < hi; ++j)
        {
            long double c, s;
            unit_root((j << shift) % L, L, c, s);
            h.push(c, s);
        }
    });
}

// e^{-2 pi i j/(2 half)}, j in [0, half/2]
static TablePtr half_twiddles(uint64_t half, int precision, bool dry)
{
    std::ostringstream key;
    key << "half_" << half;
    return cached_table(key.str(), precision, dry, [&](HostTable& h) {
        for(uint64_t j = 0; j <= half / 2; ++j)
        {
            long double c, s;
            unit_root(j, 2 * half, c, s);
            h.push(c, s);
        }
    });
}

static void chirp_value(uint64_t m, uint64_t N, long double& c, long double& s)
{
    // e^{+i pi m^2/N} with m^2 reduced mod 2N exactly
    unsigned __int128 sq = (unsigned __int128)m * m;
    uint64_t          u  = (uint64_t)(sq % (2 * (unsigned __int128)N));
    unit_root(u, 2 * N, c, s);
    s = -s;
}

static TablePtr chirp_table(uint64_t N, int precision, bool dry)
{
    std::ostringstream key;
    key << "chirp_" << N;
    return cached_table(key.str(), precision, dry, [&](HostTable& h) {
        h.v.resize(2 * N);
        host_parallel(N, [&](uint64_t first, uint64_t last) {
            for(uint64_t m = first; m < last; ++m)
                chirp_value(m, N, h.v[2 * m], h.v[2 * m + 1]);
        });
    });
}

// ---------------------------------------------------------------------------
// factorisation

static bool factorize(uint64_t n, std::vector<uint32_t>& radix, bool composite = true)
{
    radix.clear();
    if(n <= 1)
        return n == 1;
    static const uint32_t odd[] = {17, 13, 11, 7};
    uint64_t              m     = n;
    for(uint32_t r : odd)
        while(m % r == 0)
        {
            radix.push_back(r);
            m /= r;
        }
    uint32_t k = 0, threes = 0, fives = 0;
    while(m % 5 == 0)
    {
        ++fives;
        m /= 5;
    }
    while(m % 3 == 0)
    {
        ++threes;
        m /= 3;
    }
    while(m % 2 == 0)
    {
        ++k;
        m /= 2;
    }
    if(m != 1)
        return false;
    // composite butterflies save passes: 3*3 -> 9, then 5*2 -> 10 and 3*2 -> 6 while twos remain
    for(; composite && threes >= 2; threes -= 2)
        radix.push_back(9);
    for(; fives > 0; --fives)
        if(composite && k > 0)
        {
            radix.push_back(10);
            --k;
        }
        else
            radix.push_back(5);
    for(; threes > 0; --threes)
    {
        if(composite && k > 0)
        {
            radix.push_back(6);
            --k;
        }
        else
            radix.push_back(3);
    }
    // 2^k as radix-16 passes plus one or two smaller ones
    uint32_t a = k / 4, b = k % 4;
    std::vector<uint32_t> two;
    if(b == 1 && a >= 1)
    {
        --a;
        two.push_back(8);
        two.push_back(4);
    }
    else if(b == 1)
        two.push_back(2);
    else if(b == 2)
        two.push_back(4);
    else if(b == 3)
        two.push_back(8);
    for(uint32_t i = 0; i < a; ++i)
        radix.push_back(16);
    for(uint32_t r : two)
        radix.push_back(r);
    return radix.size() <= FFTK_MAX_PASSES;
}

static uint32_t threads_per_transform(uint64_t n, const std::vector<uint32_t>& radix)
{
    uint32_t T = 1;
    for(uint32_t r : radix)
    {
        uint32_t m     = (uint32_t)(n / r);
        uint32_t slots = FFTK_REG_ELEMS / r;
        T              = std::max(T, (m + slots - 1) / slots);
    }
    return T;
}

static uint32_t lds_pitch(uint32_t n)
{
    uint32_t p = n + ((n - 1) >> PADSHIFT) + 1;
    return p | 1u; // odd, so neighbouring transforms start in different banks
}

// Pass schedule of a tile kernel for length n: the one of the compile-time-schedule kernel
// when the runtime has one for this length, else the planner's own factorisation.  Returns
// the threads per transform (0: no schedule); *fast tells which kind it is.
static uint32_t kernel_schedule(uint64_t n, int precision, std::vector<uint32_t>& radix, bool* fast)
{
    radix.clear();
    if(fast)
        *fast = false;
    if(n < 1 || n > 65536)
        return 0;
    if(g_use_fast)
    {
        uint32_t fr[FFTK_MAX_PASSES] = {0}, fnf = 0;
        uint32_t tpt = fftrt_fast_schedule(precision, (uint32_t)n, fr, &fnf);
        if(tpt && fnf >= 1 && fnf <= 4)
        {
            radix.assign(fr, fr + fnf);
            if(fast)
                *fast = true;
            return tpt;
        }
    }
    // composite radices save passes but want more threads; fall back to prime radices when
    // that is what fits a workgroup
    if(factorize(n, radix, true))
    {
        uint32_t T = threads_per_transform(n, radix);
        if(T <= MAX_THREADS)
            return T;
    }
    if(!factorize(n, radix, false))
        return 0;
    return threads_per_transform(n, radix);
}

// can a single tile kernel transform length n (one transform per workgroup at least)?
static bool single_kernel_length(uint64_t n, size_t elem_bytes)
{
    std::vector<uint32_t> radix;
    uint32_t              T = kernel_schedule(n, elem_bytes == 16 ? 1 : 0, radix, nullptr);
    if(T == 0 || T > MAX_THREADS)
        return false;
    return (size_t)lds_pitch((uint32_t)n) * elem_bytes <= LDS_HARD_BYTES;
}

// Lengths that only a compiled kernel with more than MAX_THREADS threads per transform can
// take in one pass (no generic-kernel fallback exists for them: the pass must be able to use
// the kernel's lean variant).
static bool wide_kernel_length(uint64_t n, size_t elem_bytes)
{
    std::vector<uint32_t> radix;
    bool                  fast = false;
    uint32_t              T    = kernel_schedule(n, elem_bytes == 16 ? 1 : 0, radix, &fast);
    if(!fast || T <= MAX_THREADS || T > WIDE_THREADS)
        return false;
    return (size_t)lds_pitch((uint32_t)n) * elem_bytes <= LDS_HARD_BYTES;
}

// longest length a strided pass handles while keeping COL_RUN_BYTES contiguous per row
static bool column_kernel_length(uint64_t n, size_t elem_bytes)
{
    if(!single_kernel_length(n, elem_bytes))
        return false;
    size_t w = std::max<size_t>(1, COL_RUN_BYTES / elem_bytes);
    return (size_t)lds_pitch((uint32_t)n) * elem_bytes * w <= LDS_COL_BYTES;
}

static uint32_t floor_pow2(uint64_t v)
{
    uint32_t p = 1;
    while((uint64_t)p * 2 <= v)
        p *= 2;
    return p;
}
// widest tile (transforms per workgroup) a strided pass over length n can have: bounded by
// the 512 threads of a workgroup and by LDS_WIDE_BYTES
static uint32_t widest_column_tile(uint64_t n, size_t elem_bytes)
{
    std::vector<uint32_t> radix;
    uint32_t              T = kernel_schedule(n, elem_bytes == 16 ? 1 : 0, radix, nullptr);
    if(T == 0 || T > MAX_THREADS)
        return 0;
    size_t per_tile = (size_t)lds_pitch((uint32_t)n) * elem_bytes;
    if(per_tile > LDS_WIDE_BYTES)
        return 0;
    return std::min(floor_pow2(MAX_THREADS / T), floor_pow2(LDS_WIDE_BYTES / per_tile));
}

// May a whole strided dimension of length n (strides is/os scalars between its elements) run
// as one strided pass even though its tile cannot keep COL_RUN_BYTES per row?  Measured on
// MI355X: one pass with 64-byte rows beats two passes, and so does one with 32-byte rows
// unless the stride is a multiple of 512 bytes (rows a power-of-two stride apart alias onto
// the same HBM channels).
static bool narrow_column_ok(uint64_t n, size_t elem_bytes, int64_t is, int64_t os)
{
    if(is <= 0 || os <= 0)
        return false;
    const size_t wmax = widest_column_tile(n, elem_bytes);
    // the tile spans everything that lies between two elements of the dimension: its rows are
    // whole contiguous runs, however short
    if(wmax > 0 && (int64_t)(2 * wmax) >= is && (int64_t)(2 * wmax) >= os)
        return true;
    const size_t run     = wmax * elem_bytes;
    const size_t scalar  = elem_bytes / 2;
    const bool   aligned = ((size_t)is * scalar) % 512 == 0 || ((size_t)os * scalar) % 512 == 0;
    return run >= 64 || (!aligned && run >= 32);
}

static uint32_t ceil_pow2(uint64_t v)
{
    uint32_t p = 1;
    while(p < v)
        p *= 2;
    return p;
}
static uint32_t log2u(uint32_t v)
{
    uint32_t s = 0;
    while((1u << s) < v)
        ++s;
    return s;
}

// ---------------------------------------------------------------------------
// views: a logical array with up to three dimensions plus batch, strides in scalars

struct View
{
    IoRef   io;
    int64_t stride[4] = {0, 0, 0, 0};
};

static View complex_view(int buf, rocfft_array_type type, const size_t* stride, size_t dist,
                         const size_t* offset, size_t rank)
{
    View v;
    v.io.buf    = buf;
    bool planar = type == rocfft_array_type_complex_planar || type == rocfft_array_type_hermitian_planar;
    v.io.planar = planar;
    int64_t m   = planar ? 1 : 2;
    v.io.im_delta = 1;
    v.io.off0     = m * (int64_t)offset[0];
    v.io.off1     = planar ? (int64_t)offset[1] : 0;
    for(size_t d = 0; d < 3; ++d)
        v.stride[d] = d < rank ? m * (int64_t)stride[d] : 0;
    v.stride[3] = m * (int64_t)dist;
    return v;
}

// real array seen as complex pairs along dimension 0 (even-length real transforms)
static View realpair_view(int buf, const size_t* stride, size_t dist, const size_t* offset,
                          size_t rank)
{
    View v;
    v.io.buf      = buf;
    v.io.planar   = false;
    v.io.im_delta = (int64_t)stride[0];
    v.io.off0     = (int64_t)offset[0];
    for(size_t d = 0; d < 3; ++d)
        v.stride[d] = d < rank ? (int64_t)stride[d] : 0;
    v.stride[0] *= 2;
    v.stride[3] = (int64_t)dist;
    return v;
}

// real array, one scalar per element
static View real_view(int buf, const size_t* stride, size_t dist, const size_t* offset, size_t rank)
{
    View v;
    v.io.buf      = buf;
    v.io.planar   = false;
    v.io.im_delta = 0;
    v.io.off0     = (int64_t)offset[0];
    for(size_t d = 0; d < 3; ++d)
        v.stride[d] = d < rank ? (int64_t)stride[d] : 0;
    v.stride[3] = (int64_t)dist;
    return v;
}

// ---------------------------------------------------------------------------
// tile pass construction

struct Axis
{
    uint32_t cnt;
    int64_t  is, os;
    bool     aux;
    uint32_t aux_shift = 0; // aux axis with a faster plain axis merged in: table index = index >> aux_shift
};

struct TileSpec
{
    uint32_t          n        = 1;
    int64_t           t_is = 0, t_os = 0;
    std::vector<Axis> others;
    IoRef             src, dst;
    int64_t           src_extra = 0, dst_extra = 0; // extra scalar offsets
    uint32_t          load_op = FFTK_LOAD_COMPLEX, store_op = FFTK_STORE_COMPLEX;
    uint32_t          flags = 0;
    int               dir   = -1;
    uint32_t          n_in = 0, n_out = 0; // 0 = n
    TablePtr          ltw, half_tw, chirp, convb;
    uint32_t          ltw_shift = 0;
    uint32_t          ltw_qmul = 1, ltw_qadd = 0; // twiddle of output j: W^{j (q ltw_qmul + ltw_qadd)}
    uint32_t          blu_n = 0, chirp_js = 0, chirp_qs = 0, convb_qs = 0;
    uint64_t          convb_off = 0; // first element of the chirp spectrum this pass reads
    double            scale = 1.0;
    std::string       note;
    bool              src_real_scalar = false, dst_real_scalar = false;
};

static bool io_vec_ok(const IoRef& io, bool real_scalar)
{
    return !io.planar && !real_scalar && io.im_delta == 1 && (io.off0 % 2 == 0);
}

static PassRec make_tile_pass(const TileSpec& s, int precision, bool dry)
{
    const size_t esize = precision ? 16 : 8;
    PassRec      rec;
    rec.kind = PASS_TILE;
    rec.src  = s.src;
    rec.dst  = s.dst;
    rec.src.off0 += s.src_extra;
    rec.src.off1 += s.src_extra;
    rec.dst.off0 += s.dst_extra;
    rec.dst.off1 += s.dst_extra;
    rec.note = s.note;

    fftk_params& k = rec.kp;
    memset(&k, 0, sizeof(k));
    k.n = s.n;
    std::vector<uint32_t> radix;
    bool                  have_fast = false;
    const uint32_t        sched_T   = kernel_schedule(s.n, precision, radix, &have_fast);
    if(sched_T == 0)
        fail("length has no kernel factorisation");
    k.nf         = (uint32_t)radix.size();
    uint32_t cum = 1;
    for(size_t p = 0; p < radix.size(); ++p)
    {
        k.radix[p]  = radix[p];
        k.cum[p]    = cum;
        k.cshift[p] = (cum & (cum - 1)) == 0 ? log2u(cum) : 0xff;
        cum *= radix[p];
    }
    TablePtr tw = stacked_twiddles(radix, precision, dry, k.twoff);
    k.tw        = tw->dptr;
    rec.tables.push_back(tw);

    // drop unit axes, merge axes that continue one another
    std::vector<Axis> ax;
    for(const Axis& a : s.others)
        if(a.cnt > 1 || a.aux)
            ax.push_back(a);
    for(bool merged = true; merged;)
    {
        merged = false;
        for(size_t i = 0; i < ax.size() && !merged; ++i)
            for(size_t j = 0; j < ax.size() && !merged; ++j)
            {
                if(i == j || ax[i].aux)
                    continue;
                // a plain axis may also merge into the table-indexed (aux) axis it continues into,
                // when its length is a power of two: the table index is then the merged index
                // shifted right
                if(ax[j].aux && (ax[j].aux_shift || (ax[i].cnt & (ax[i].cnt - 1)) || ax[i].cnt < 2))
                    continue;
                if(ax[i].is * (int64_t)ax[i].cnt == ax[j].is && ax[i].os * (int64_t)ax[i].cnt == ax[j].os
                   && (uint64_t)ax[i].cnt * ax[j].cnt < (1ull << 31))
                {
                    if(ax[j].aux)
                    {
                        ax[i].aux       = true;
                        ax[i].aux_shift = log2u(ax[i].cnt);
                    }
                    ax[i].cnt *= ax[j].cnt;
                    ax.erase(ax.begin() + (long)j);
                    merged = true;
                }
            }
    }
    if(ax.size() > 4)
        fail("too many independent dimensions for one pass");

    // tile axis: the one global accesses should run along when the transform axis is strided
    int     tile = -1;
    int64_t best = 0;
    auto    pick = [&](bool by_in) {
        for(size_t i = 0; i < ax.size(); ++i)
        {
            int64_t st = by_in ? ax[i].is : ax[i].os;
            if(tile < 0 || st < best)
            {
                tile = (int)i;
                best = st;
            }
        }
    };
    bool row_in = true, row_out = true;
    for(const Axis& a : ax)
    {
        if(a.cnt > 1 && a.is < s.t_is)
            row_in = false;
        if(a.cnt > 1 && a.os < s.t_os)
            row_out = false;
    }
    if(!ax.empty())
    {
        if(!row_in)
            pick(true);
        else if(!row_out)
            pick(false);
        else
            pick(true);
    }
    Axis tile_axis = {1, 0, 0, false};
    if(tile >= 0)
    {
        tile_axis = ax[(size_t)tile];
        ax.erase(ax.begin() + tile);
    }
    if(ax.size() > 3)
        fail("too many independent dimensions for one pass");
    k.tile_cnt      = tile_axis.cnt;
    k.w_is          = tile_axis.is;
    k.w_os          = tile_axis.os;
    k.t_is          = s.t_is;
    k.t_os          = s.t_os;
    k.in_fast_tile  = (tile_axis.cnt > 1 && tile_axis.is < s.t_is) ? 1 : 0;
    k.out_fast_tile = (tile_axis.cnt > 1 && tile_axis.os < s.t_os) ? 1 : 0;
    k.aux_dim       = tile_axis.aux ? 1 : 0;
    k.aux_shift     = tile_axis.aux ? tile_axis.aux_shift : 0;
    // A column pass over very short rows (a 4 x 5 transform: 4 columns) would leave most lanes of
    // its workgroups idle.  Fold the longest other plain axis (the transforms of a batch) into the
    // tile axis: tile entries are then (column, batch item) pairs.
    // (Only where the tiles would otherwise not fill one wave, or run less than 65 % full: a row
    // count just below a power of two, or many threads per transform, keep the workgroups busy
    // anyway, and folding measured 0-25 % slower there.)
    bool fold_pays = false;
    {
        const uint32_t w_plain = std::min<uint32_t>(std::min<uint32_t>(64, floor_pow2(std::max<uint32_t>(1, 512 / sched_T))),
                                                    ceil_pow2(tile_axis.cnt));
        const uint64_t slots   = (uint64_t)((tile_axis.cnt + w_plain - 1) / w_plain) * w_plain;
        fold_pays = (uint64_t)w_plain * sched_T < 64 || (double)tile_axis.cnt < 0.65 * (double)slots;
    }
    if(g_fold_tiles && (k.in_fast_tile || k.out_fast_tile) && !tile_axis.aux && fold_pays && tile_axis.cnt < 64
       && tile_axis.is >= 0 && tile_axis.os >= 0)
    {
        int fold = -1;
        for(size_t i = 0; i < ax.size(); ++i)
            if(!ax[i].aux && ax[i].cnt > 1 && ax[i].is >= 0 && ax[i].os >= 0
               && (fold < 0 || ax[i].cnt > ax[(size_t)fold].cnt))
                fold = (int)i;
        if(fold >= 0 && (uint64_t)tile_axis.cnt * ax[(size_t)fold].cnt < (1ull << 31))
        {
            k.w_inner  = tile_axis.cnt;
            k.w2_is    = ax[(size_t)fold].is;
            k.w2_os    = ax[(size_t)fold].os;
            k.tile_cnt = tile_axis.cnt * ax[(size_t)fold].cnt;
            ax.erase(ax.begin() + fold);
        }
    }
    for(int i = 0; i < 3; ++i)
    {
        k.oc[i]   = 1;
        k.o_is[i] = k.o_os[i] = 0;
    }
    // A pass that multiplies by a long table (chirp, chirp spectrum) indexes it with the tile or
    // an outer axis; the remaining plain axis (the signals of a batch) re-reads the same entries.
    // That axis goes first in the workgroup numbering, so that the re-reads follow one another.
    // (Tables beyond a megabyte only: shorter ones stay in L2 anyway.  One outer axis only: with
    // more, neighbouring column tiles would no longer be neighbours in the numbering.)
    bool         shared_table_axis = false;
    const size_t table_bytes       = std::max(s.chirp ? s.chirp->bytes : 0, s.convb ? s.convb->bytes : 0);
    if(table_bytes >= (1u << 20) && ax.size() == 1 && !ax[0].aux && ax[0].cnt > 1)
        shared_table_axis = true;
    for(size_t i = 0; i < ax.size(); ++i)
    {
        k.oc[i]   = ax[i].cnt;
        k.o_is[i] = ax[i].is;
        k.o_os[i] = ax[i].os;
        if(ax[i].aux)
        {
            k.aux_dim   = 2 + (uint32_t)i;
            k.aux_shift = ax[i].aux_shift;
        }
    }

    // work split
    k.T        = sched_T;
    k.padshift = PADSHIFT;
    k.pitch    = lds_pitch(s.n);
    if(k.T > MAX_THREADS && !(have_fast && k.T <= WIDE_THREADS))
        fail("transform too long for one workgroup");
    // a kernel compiled for exactly this pass schedule, when there is one
    uint32_t max_threads = MAX_THREADS;
    uint32_t fast_tpt    = have_fast ? sched_T : 0;
    if(fast_tpt)
    {
        k.fast      = 1;
        k.T         = fast_tpt;
        // a strided pass may use the larger workgroup to keep its tile rows wide
        max_threads = fast_tpt > 512 ? WIDE_THREADS
                                     : (fast_tpt > 256 || k.in_fast_tile || k.out_fast_tile) ? 512 : 256;
    }
    size_t   per_tile  = (size_t)k.pitch * esize;
    uint32_t w_threads = floor_pow2(max_threads / k.T);
    uint32_t w_lds     = per_tile <= LDS_SOFT_BYTES ? floor_pow2(LDS_SOFT_BYTES / per_tile) : 1;
    if(per_tile > LDS_HARD_BYTES)
        fail("transform too long for the LDS of one compute unit");
    uint32_t w_cap  = ceil_pow2(k.tile_cnt);
    bool     column = k.in_fast_tile || k.out_fast_tile;
    uint32_t W;
    if(column)
    {
        // keep COL_RUN_BYTES contiguous per tile row even if that costs occupancy
        uint32_t w_run = (uint32_t)std::max<size_t>(1, COL_RUN_BYTES / esize);
        if(w_lds < w_run && per_tile * w_run <= LDS_COL_BYTES)
            w_lds = w_run;
        else if(w_lds < w_run && per_tile <= LDS_WIDE_BYTES)
            w_lds = std::max(w_lds, std::min(w_run, floor_pow2(LDS_WIDE_BYTES / per_tile)));
        W = std::min(std::min<uint32_t>(64, w_threads), std::min(w_lds, w_cap));
        // experiment switch: ROCFFT_AMD_COLW=<w> asks for column tiles w transforms wide (when
        // threads and LDS allow)
        static const char* colw = getenv("ROCFFT_AMD_COLW");
        if(colw)
        {
            const uint32_t want = (uint32_t)atoi(colw);
            const uint32_t fit  = std::min(w_threads, floor_pow2((uint32_t)(LDS_WIDE_BYTES / per_tile)));
            if(want >= 1)
                W = std::min(std::min(want, fit), w_cap);
        }
    }
    else
    {
        uint32_t target = floor_pow2(std::max<uint32_t>(1, 256 / k.T));
        W               = std::min(std::min(target, w_threads), std::min(w_lds, w_cap));
    }
    W          = std::max<uint32_t>(W, 1);
    k.W        = W;
    k.wshift   = log2u(W);
    k.wfast    = W >= 16 ? 1 : 0;
    if(k.fast)
    {
        // lanes follow the fast axis of the input; a side whose fast axis differs, or whose
        // fused operation needs partner elements, is staged through LDS
        k.wfast      = k.in_fast_tile;
        k.direct_in  = s.load_op != FFTK_LOAD_C2R_PRE ? 1 : 0;
        k.direct_out = (s.store_op != FFTK_STORE_R2C_POST && k.out_fast_tile == k.in_fast_tile) ? 1 : 0;
    }
    k.nthreads = (k.T * W + 63) / 64 * 64;
    rec.lds    = (size_t)k.pitch * W * esize;
    uint64_t ntile = (k.tile_cnt + W - 1) / W;
    uint64_t grid  = ntile * k.oc[0] * k.oc[1] * k.oc[2];
    if(grid == 0 || grid >= (1ull << 31))
        fail("grid too large");
    rec.grid = (uint32_t)grid;
    k.grid      = rec.grid;
    // Neighbouring column tiles share 128-byte lines when the rows of the array are not
    // line-aligned; then each XCD should own a contiguous range of tiles.
    {
        const int64_t line  = 128 / (precision ? 8 : 4); // scalars per 128 bytes
        const bool    split = (k.in_fast_tile && (k.t_is % line)) || (k.out_fast_tile && (k.t_os % line));
        k.xcd_remap         = (g_xcd_remap && column && split && rec.grid >= 64) ? 1 : 0;
    }
    if(shared_table_axis && g_share_first)
    {
        k.oc0_first = 1;
        k.xcd_remap = (g_xcd_remap && rec.grid >= 64) ? 1 : 0;
    }

    k.flags    = s.flags;
    k.dir      = s.dir;
    k.load_op  = s.load_op;
    k.store_op = s.store_op;
    k.n_in     = s.n_in ? s.n_in : s.n;
    k.n_out    = s.n_out ? s.n_out : s.n;
    if(s.ltw)
    {
        k.ltw       = s.ltw->dptr;
        k.ltw_shift = s.ltw_shift;
        k.ltw_qmul  = s.ltw_qmul;
        k.ltw_qadd  = s.ltw_qadd;
        rec.tables.push_back(s.ltw);
    }
    if(s.half_tw)
    {
        k.half_tw = s.half_tw->dptr;
        rec.tables.push_back(s.half_tw);
    }
    if(s.chirp)
    {
        k.chirp    = s.chirp->dptr;
        k.blu_n    = s.blu_n;
        k.chirp_js = s.chirp_js;
        k.chirp_qs = s.chirp_qs;
        rec.tables.push_back(s.chirp);
    }
    if(s.convb)
    {
        k.convb    = s.convb->dptr ? static_cast<const char*>(s.convb->dptr) + s.convb_off * esize : nullptr;
        k.convb_qs = s.convb_qs;
        rec.tables.push_back(s.convb);
    }
    k.scale = s.scale;

    // one access per (re, im) pair needs interleaved data with even scalar strides
    bool vec = io_vec_ok(rec.src, s.src_real_scalar) && io_vec_ok(rec.dst, s.dst_real_scalar);
    auto even = [](int64_t v) { return v % 2 == 0; };
    vec = vec && even(k.t_is) && even(k.t_os) && even(k.w_is) && even(k.w_os) && even(k.w2_is) && even(k.w2_os);
    for(int i = 0; i < 3; ++i)
        vec = vec && even(k.o_is[i]) && even(k.o_os[i]);
    if(s.load_op == FFTK_LOAD_REAL || s.store_op == FFTK_STORE_REAL)
        vec = false;
    rec.vec_ok = vec;
    // branch-free addressing path of the fast kernel: complex arrays on both sides (real pairs
    // with unit real stride count), element offsets inside a tile fit 32 bits.  A side is
    // interleaved (even scalar strides) or planar (scalar strides are element strides).
    auto even_side = [&](bool in) {
        bool ok = in ? (even(k.t_is) && even(k.w_is) && even(k.w2_is)) : (even(k.t_os) && even(k.w_os) && even(k.w2_os));
        for(int i = 0; i < 3; ++i)
            ok = ok && even(in ? k.o_is[i] : k.o_os[i]);
        return ok;
    };
    // largest offset of a tile entry from the tile's base, for strides w (and w2 of a folded axis)
    auto tile_extent = [&](int64_t w, int64_t w2) -> uint64_t {
        if(!k.w_inner)
            return (uint64_t)W * (uint64_t)w;
        return ((uint64_t)(W + k.w_inner - 1) / k.w_inner + 1) * (uint64_t)w2 + (uint64_t)k.w_inner * (uint64_t)w;
    };
    // element offsets inside a tile are 32-bit: their byte offsets must be too
    const uint64_t lean_span_limit = (1ull << 32) / esize;
    // 0: no lean access, 1: interleaved, 2: planar, 3: real scalars
    auto side_kind = [&](const IoRef& io, bool real_scalar, bool in) {
        if(io.planar)
            return real_scalar ? 0 : 2;
        if(real_scalar)
            return 3;
        return io_vec_ok(io, real_scalar) && even_side(in) ? 1 : 0;
    };
    int in_kind = side_kind(rec.src, s.src_real_scalar, true), out_kind = side_kind(rec.dst, s.dst_real_scalar, false);
    // real sides: only together with the Bluestein chirp of that side (odd-length real transforms of
    // lengths with large prime factors); the plain odd-length real kernels follow below
    const bool chirp_rows = (k.flags & FFTK_F_CHIRP_LOAD) && k.chirp_js == 1 && k.chirp_qs == 0 && k.n_in == k.blu_n;
    if((in_kind == 3) != (s.load_op == FFTK_LOAD_REAL) || (in_kind == 3 && !chirp_rows))
        in_kind = 0;
    if((out_kind == 3) != (s.store_op == FFTK_STORE_REAL) || (out_kind == 3 && !(k.flags & FFTK_F_CHIRP_STORE)))
        out_kind = 0;
    {
        const uint32_t lean_flags = FFTK_F_TWIDDLE_STORE | FFTK_F_SCALE | FFTK_F_CHIRP_LOAD
                                    | FFTK_F_CHIRP_STORE | FFTK_F_CHIRP_CONJ | FFTK_F_CONV;
        bool ops_ok = (s.load_op == FFTK_LOAD_COMPLEX || s.load_op == FFTK_LOAD_C2R_PRE || in_kind == 3
                       || (s.load_op == FFTK_LOAD_HERM_EXPAND && chirp_rows))
                      && (s.store_op == FFTK_STORE_COMPLEX || s.store_op == FFTK_STORE_R2C_POST || out_kind == 3)
                      && (k.flags & ~lean_flags) == 0;
        // short inputs/outputs are only expressed through the chirp index test
        if(k.n_in != k.n && !((k.flags & FFTK_F_CHIRP_LOAD) && k.chirp_js == 1 && k.chirp_qs == 0
                              && k.n_in == k.blu_n))
            ops_ok = false;
        if(k.n_out != k.n && !(k.flags & FFTK_F_CHIRP_STORE))
            ops_ok = false;
        if(s.load_op == FFTK_LOAD_C2R_PRE && (k.flags & (FFTK_F_CHIRP_LOAD | FFTK_F_CONV)))
            ops_ok = false;
        if(s.store_op == FFTK_STORE_R2C_POST && (k.flags & (FFTK_F_CHIRP_STORE | FFTK_F_TWIDDLE_STORE)))
            ops_ok = false;
        if(k.fast && in_kind && out_kind && ops_ok && k.t_is >= 0 && k.t_os >= 0 && k.w_is >= 0 && k.w_os >= 0)
        {
            const int64_t in_div = in_kind == 1 ? 2 : 1, out_div = out_kind == 1 ? 2 : 1;
            uint64_t in_span  = (uint64_t)(k.n + 1) * (uint64_t)(k.t_is / in_div) + tile_extent(k.w_is / in_div, k.w2_is / in_div);
            uint64_t out_span = (uint64_t)(k.n + 1) * (uint64_t)(k.t_os / out_div) + tile_extent(k.w_os / out_div, k.w2_os / out_div);
            if(in_span < lean_span_limit && out_span < lean_span_limit)
            {
                rec.lean_ok    = true;
                k.in_planar    = in_kind == 2;
                k.out_planar   = out_kind == 2;
                // short transforms in unit-stride rows: coalesced tile copies through LDS
                // (also the fused real pre/post-processing: rows of n+1 bins on that side)
                const bool plain_ops = s.load_op == FFTK_LOAD_COMPLEX && s.store_op == FFTK_STORE_COMPLEX;
                const bool real_ops  = (s.load_op == FFTK_LOAD_COMPLEX && s.store_op == FFTK_STORE_R2C_POST)
                                      || (s.load_op == FFTK_LOAD_C2R_PRE && s.store_op == FFTK_STORE_COMPLEX);
                // (lanes of a transform that together cover 16 bytes or less per access)
                const size_t access = (in_kind == 2 || out_kind == 2) ? esize / 2 : esize;
                if(!column && (k.T == 1 || ((size_t)k.T * access <= 16 && k.n < 32)) && k.t_is == (in_kind == 1 ? 2 : 1)
                   && k.t_os == (out_kind == 1 ? 2 : 1) && in_kind <= 2 && out_kind <= 2
                   && (plain_ops || real_ops) && (k.flags & ~(uint32_t)FFTK_F_SCALE) == 0 && k.n_in == k.n
                   && k.n_out == k.n)
                {
                    k.stage_io = 1;
                    // the tile copy writes LDS without bounds tests: room for every element index
                    // its threads reach (rows of n, or of n + 1 bins on a Hermitian side)
                    const uint64_t it_plain = (k.n + k.T - 1) / k.T, it_bins = (k.n + 1 + k.T - 1) / k.T;
                    const uint64_t rows     = (it_plain * k.nthreads - 1) / k.n + 1;
                    rec.lds = std::max<size_t>(rec.lds, std::max<uint64_t>(rows * k.pitch, it_bins * k.nthreads) * esize);
                }
                k.t_is_c    = (uint32_t)(k.t_is / in_div);
                k.t_os_c    = (uint32_t)(k.t_os / out_div);
                k.w_is_c    = (uint32_t)(k.w_is / in_div);
                k.w_os_c    = (uint32_t)(k.w_os / out_div);
                k.w2_is_c   = (uint32_t)(k.w2_is / in_div);
                k.w2_os_c   = (uint32_t)(k.w2_os / out_div);
            }
        }
    }

    // odd-length real transforms on the same path: real samples in -> the first n/2+1 bins out,
    // or those bins in (mirrored to the full spectrum on load) -> real samples out.  The real
    // side is addressed in scalars, the complex side is interleaved with even strides or planar.
    {
        const bool fwd = s.load_op == FFTK_LOAD_REAL && s.store_op == FFTK_STORE_COMPLEX && k.n_in == k.n
                         && k.n_out == k.n / 2 + 1;
        const bool bwd = s.load_op == FFTK_LOAD_HERM_EXPAND && s.store_op == FFTK_STORE_REAL && k.n_in == k.n
                         && k.n_out == k.n;
        const int  cplx_kind = fwd ? out_kind : in_kind;
        const bool real_ok = fwd ? !rec.src.planar : !rec.dst.planar;
        if(k.fast && (fwd || bwd) && (k.n & 1u) && cplx_kind && real_ok && (k.flags & ~(uint32_t)FFTK_F_SCALE) == 0
           && k.t_is >= 0 && k.t_os >= 0 && k.w_is >= 0 && k.w_os >= 0)
        {
            const int64_t cdiv = cplx_kind == 2 ? 1 : 2;
            const int64_t ti = fwd ? k.t_is : k.t_is / cdiv, wi = fwd ? k.w_is : k.w_is / cdiv;
            const int64_t to = fwd ? k.t_os / cdiv : k.t_os, wo = fwd ? k.w_os / cdiv : k.w_os;
            uint64_t      in_span  = (uint64_t)(k.n + 1) * (uint64_t)ti + tile_extent(wi, fwd ? k.w2_is : k.w2_is / cdiv);
            uint64_t      out_span = (uint64_t)(k.n + 1) * (uint64_t)to + tile_extent(wo, fwd ? k.w2_os / cdiv : k.w2_os);
            if(in_span < lean_span_limit && out_span < lean_span_limit)
            {
                rec.lean_ok = true;
                k.in_planar = bwd && cplx_kind == 2;
                k.out_planar = fwd && cplx_kind == 2;
                k.t_is_c    = (uint32_t)ti;
                k.w_is_c    = (uint32_t)wi;
                k.t_os_c    = (uint32_t)to;
                k.w_os_c    = (uint32_t)wo;
                k.w2_is_c   = (uint32_t)(fwd ? k.w2_is : k.w2_is / cdiv);
                k.w2_os_c   = (uint32_t)(fwd ? k.w2_os / cdiv : k.w2_os);
            }
        }
    }

    if(k.T > MAX_THREADS && !rec.lean_ok)
        fail("no kernel for a transform this long in this layout");

    // data volume of the pass: every element it loads plus every element it stores
    {
        double lines   = (double)k.tile_cnt * k.oc[0] * k.oc[1] * k.oc[2];
        double aux_cnt = 1;
        if(k.aux_dim == 1)
            aux_cnt = k.tile_cnt;
        else if(k.aux_dim >= 2)
            aux_cnt = k.oc[k.aux_dim - 2];
        double scalar   = precision ? 8 : 4;
        double in_elems = lines * std::min(k.n_in, k.n);
        if(k.load_op == FFTK_LOAD_C2R_PRE)
            in_elems = lines * (k.n + 1);
        else if(k.load_op == FFTK_LOAD_HERM_EXPAND)
            in_elems = lines * (k.n_in / 2 + 1);
        if((k.flags & FFTK_F_CHIRP_LOAD) && k.chirp_qs)
            in_elems = lines / aux_cnt * k.blu_n;
        double out_elems = lines * std::min(k.n_out, k.n);
        if(k.store_op == FFTK_STORE_R2C_POST)
            out_elems = lines * (k.n + 1);
        if((k.flags & FFTK_F_CHIRP_STORE) && k.chirp_qs)
            out_elems = lines / aux_cnt * k.blu_n;
        rec.bytes_rw = in_elems * scalar * (k.load_op == FFTK_LOAD_REAL ? 1 : 2)
                       + out_elems * scalar * (k.store_op == FFTK_STORE_REAL ? 1 : 2);
    }
    return rec;
}

// ---------------------------------------------------------------------------
// emitters

struct Builder
{
    ExecPlan* plan;
    int       precision;
    bool      dry;
    size_t    esize;
    void      need_tmp(size_t elems)
    {
        plan->tmp_elems = std::max(plan->tmp_elems, elems);
    }
    void need_cpx(size_t elems)
    {
        plan->cpx_elems = std::max(plan->cpx_elems, elems);
    }
    void need_blu(size_t elems)
    {
        plan->blu_elems = std::max(plan->blu_elems, elems);
    }
};

struct Other
{
    uint32_t cnt;
    int64_t  is, os;
};

struct DimOps
{
    // fused input/output operations of the first/last pass of the dimension
    uint32_t load_op  = FFTK_LOAD_COMPLEX;
    uint32_t store_op = FFTK_STORE_COMPLEX;
    uint32_t n_in     = 0; // logical input length (0 = n)
    uint32_t n_out    = 0; // outputs kept (0 = n)
    bool     src_real_scalar = false, dst_real_scalar = false;
    TablePtr half_tw;
    double   scale     = 1.0;
    bool     has_scale = false;
};

static std::string dims_note(const char* what, uint64_t n)
{
    std::ostringstream o;
    o << what << " n=" << n;
    return o.str();
}

static void split_length(uint64_t n, size_t esize, bool column, uint64_t& n1, uint64_t& n0)
{
    // n = n1 * n0, both single-kernel lengths, as balanced as possible; n0 is the
    // length of the pass that reads rows of the intermediate array
    uint64_t best = 0;
    double   root = std::sqrt((double)n);
    for(uint64_t a = 2; a * a <= n; ++a)
    {
        if(n % a)
            continue;
        uint64_t b  = n / a;
        auto     ok = [&](uint64_t v) {
            return column ? column_kernel_length(v, esize) : single_kernel_length(v, esize);
        };
        if(!ok(a) || !ok(b))
            continue;
        if(best == 0 || std::fabs((double)a - root) < std::fabs((double)best - root))
            best = a;
    }
    if(best == 0)
    {
        n1 = n0 = 0;
        return;
    }
    n1 = best;
    n0 = n / best;
}

static void split_length(uint64_t n, size_t esize, bool column, uint64_t& n1, uint64_t& n0);

static bool factorize(uint64_t n, std::vector<uint32_t>& radix, bool composite);

static bool fast_kernel_exists(uint64_t n, size_t esize)
{
    std::vector<uint32_t> radix;
    bool                  fast = false;
    kernel_schedule(n, esize == 16 ? 1 : 0, radix, &fast);
    return fast;
}

// Will emit_dim transform a plain complex dimension of length n with one tile pass?
// is/os: scalar strides of the dimension on both sides (0 = not known)
static bool plain_dim_is_single(uint64_t n, bool column, size_t esize, int64_t is, int64_t os)
{
    bool single = column ? (column_kernel_length(n, esize) || narrow_column_ok(n, esize, is, os))
                         : single_kernel_length(n, esize);
    // Longer lengths without a compile-time-schedule kernel (most above 4096, 5^5 below): two
    // passes of those kernels beat one pass of the run-time-schedule kernel, so split them
    // when both factors have one.
    if(single && g_use_fast && n >= 1024 && !fast_kernel_exists(n, esize))
    {
        uint64_t a1, a0;
        split_length(n, esize, column, a1, a0);
        if(a1 != 0 && ((n > 4096 && (n & (n - 1)) == 0)
                       || (fast_kernel_exists(a1, esize) && fast_kernel_exists(a0, esize))))
            single = false;
    }
    return single;
}

// n = n1 * n0 for the two-pass scheme: pass A is a strided pass over n1 (it wants a wide
// tile, so n1 must be a column-kernel length), pass B a row pass over n0 (or another strided
// pass when the whole dimension is strided).  Prefers factors with compile-time-schedule
// kernels, then balance.  n1 = 0 when there is no such pair.
static void split_two(uint64_t n, size_t esize, bool column, uint64_t& n1, uint64_t& n0,
                      uint64_t max_row = 8192)
{
    n1 = n0 = 0;
    double best_score = -1;
    for(uint64_t a = 2; a < n; ++a)
    {
        if(n % a)
            continue;
        uint64_t bq = n / a;
        if(!column_kernel_length(a, esize))
            continue;
        if(!(column ? column_kernel_length(bq, esize) : single_kernel_length(bq, esize)))
            continue;
        if(!column && bq > max_row)
            continue;
        double score = (fast_kernel_exists(a, esize) ? 2.0 : 0.0) + (fast_kernel_exists(bq, esize) ? 2.0 : 0.0);
        // balance: prefer a close to sqrt(n) but never a tiny strided factor
        double ratio = (double)std::min(a, bq) / (double)std::max(a, bq);
        score += ratio;
        if(a < 8)
            score -= 1.0;
        // a strided pass whose tile the thread count keeps narrow (many threads per transform)
        // moves short runs
        auto narrow = [&](uint64_t len) {
            const size_t run = (size_t)widest_column_tile(len, esize) * esize;
            return run < 64 ? 2.0 : run < COL_RUN_BYTES ? 1.0 : 0.0;
        };
        score -= narrow(a);
        if(column)
            score -= narrow(bq);
        // ... and short runs a multiple of 512 bytes apart alias onto the same HBM channels
        if(narrow(a) > 0 && (bq * esize) % 512 == 0)
            score -= 0.5;
        if(score > best_score)
        {
            best_score = score;
            n1         = a;
            n0         = bq;
        }
    }
}

// n = n2 * n1 * n0 for the three-pass scheme (n2 and n1 strided passes, n0 as in split_two)
static void split_three(uint64_t n, size_t esize, bool column, uint64_t& n2, uint64_t& n1,
                        uint64_t& n0)
{
    n2 = n1 = n0 = 0;
    double best_score = -1;
    for(uint64_t a = 2; a < n; ++a)
    {
        if(n % a || !column_kernel_length(a, esize))
            continue;
        uint64_t b1, b0;
        split_two(n / a, esize, column, b1, b0, 512);
        if(b1 == 0)
            split_two(n / a, esize, column, b1, b0);
        if(b1 == 0)
            continue;
        double score = (fast_kernel_exists(a, esize) ? 2.0 : 0.0) + (fast_kernel_exists(b1, esize) ? 2.0 : 0.0)
                       + (fast_kernel_exists(b0, esize) ? 2.0 : 0.0);
        // the long factor goes to the row pass; the two strided factors should be similar
        score += (double)std::min(a, b1) / (double)std::max(a, b1) + (double)b0 / (double)n;
        if(a < 8)
            score -= 1.0;
        if(score > best_score)
        {
            best_score = score;
            n2         = a;
            n1         = b1;
            n0         = b0;
        }
    }
}

// n = n3 * n2 * n1 * n0 for the four-pass scheme: one more strided factor outside split_three
static void split_four(uint64_t n, size_t esize, bool column, uint64_t& n3, uint64_t& n2, uint64_t& n1,
                       uint64_t& n0)
{
    n3 = n2 = n1 = n0 = 0;
    double best_score = -1;
    for(uint64_t a = 2; a < n; ++a)
    {
        if(n % a || !column_kernel_length(a, esize))
            continue;
        uint64_t b2, b1, b0;
        split_three(n / a, esize, column, b2, b1, b0);
        if(b2 == 0)
            continue;
        double score = (fast_kernel_exists(a, esize) ? 2.0 : 0.0) + (fast_kernel_exists(b2, esize) ? 2.0 : 0.0)
                       + (fast_kernel_exists(b1, esize) ? 2.0 : 0.0) + (fast_kernel_exists(b0, esize) ? 2.0 : 0.0);
        // similar strided factors, the long one in the row pass
        const uint64_t lo = std::min(a, std::min(b2, b1)), hi = std::max(a, std::max(b2, b1));
        score += (double)lo / (double)hi + (double)b0 / (double)n;
        if(a < 8)
            score -= 1.0;
        if(score > best_score)
        {
            best_score = score;
            n3         = a;
            n2         = b2;
            n1         = b1;
            n0         = b0;
        }
    }
}

static bool smooth(uint64_t n)
{
    std::vector<uint32_t> r;
    for(uint32_t p : {2u, 3u, 5u, 7u, 11u, 13u, 17u})
        while(n % p == 0)
            n /= p;
    return n == 1;
}

static TablePtr bluestein_spectrum(Builder& b, uint64_t N, uint64_t M, uint64_t M1, uint64_t M0,
                                   bool conj_chirp, uint64_t M2 = 1);
static bool     big_eligible(const Builder& b, uint64_t n, int64_t t_is, int64_t t_os,
                             const std::vector<Other>& others, const IoRef& src, const IoRef& dst);
static void     emit_big(Builder& b, uint32_t mode, const std::vector<Other>& others, const IoRef& src,
                         const IoRef& dst, int dir, double scale, bool has_scale);

// One dimension of complex transforms: length n along an axis with scalar strides
// (t_is, t_os); `others` are the remaining index dimensions.  src and dst may be
// the same buffer: every decomposition below finishes reading src before dst is
// written, going through the work buffer where a pass cannot run in place.
static void emit_dim(Builder& b, uint64_t n, int64_t t_is, int64_t t_os, const std::vector<Other>& others,
                     const IoRef& src, const IoRef& dst, int dir, const DimOps& ops)
{
    const size_t esize = b.esize;
    uint64_t     lines = 1;
    for(const Other& o : others)
        lines *= o.cnt;

    // is the transform axis the fastest one on both sides?
    bool column = false;
    for(const Other& o : others)
        if(o.cnt > 1 && (o.is < t_is || o.os < t_os))
            column = true;
    bool plain = ops.load_op == FFTK_LOAD_COMPLEX && ops.store_op == FFTK_STORE_COMPLEX && !ops.n_in
                 && !ops.n_out;

    if(plain && !column && big_eligible(b, n, t_is, t_os, others, src, dst))
    {
        emit_big(b, 0, others, src, dst, dir, ops.scale, ops.has_scale);
        return;
    }

    auto base_spec = [&]() {
        TileSpec s;
        s.dir = dir;
        return s;
    };
    auto add_others = [&](TileSpec& s, bool in_user, bool out_user, const std::vector<int64_t>& packed) {
        for(size_t i = 0; i < others.size(); ++i)
            s.others.push_back({others[i].cnt, in_user ? others[i].is : packed[i],
                                out_user ? others[i].os : packed[i], false});
    };
    // strides of the `others` axes in a packed scratch array of line length `linelen` complex
    auto packed_strides = [&](uint64_t linelen) {
        std::vector<int64_t> p;
        int64_t              st = 2 * (int64_t)linelen;
        for(const Other& o : others)
        {
            p.push_back(st);
            st *= o.cnt;
        }
        return p;
    };
    IoRef tmp;
    tmp.buf = BUF_TMP;
    IoRef blu;
    blu.buf = BUF_BLU;

    // a pass that is not "plain" (fused real/odd handling) stays single if it fits at all
    bool single = plain ? plain_dim_is_single(n, column, esize, t_is, t_os) : single_kernel_length(n, esize);
    auto emit_single = [&]() {
        TileSpec s = base_spec();
        s.n        = (uint32_t)n;
        s.t_is     = t_is;
        s.t_os     = t_os;
        s.src      = src;
        s.dst      = dst;
        add_others(s, true, true, {});
        s.load_op         = ops.load_op;
        s.store_op        = ops.store_op;
        s.n_in            = ops.n_in;
        s.n_out           = ops.n_out;
        s.half_tw         = ops.half_tw;
        s.src_real_scalar = ops.src_real_scalar;
        s.dst_real_scalar = ops.dst_real_scalar;
        if(ops.has_scale)
        {
            s.flags |= FFTK_F_SCALE;
            s.scale = ops.scale;
        }
        s.note = dims_note(column ? "column fft" : "row fft", n);
        b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
    };
    if(single)
    {
        emit_single();
        return;
    }
    // one workgroup of up to 1024 threads, when the layout suits the compiled kernel's lean variant
    if(!column && wide_kernel_length(n, esize))
    {
        const size_t mark = b.plan->passes.size();
        try
        {
            emit_single();
            return;
        }
        catch(const PlanError&)
        {
            b.plan->passes.resize(mark);
        }
    }

    if(smooth(n))
    {
        if(!plain)
            fail("this real-transform length needs a decomposition that is not implemented");
        // The row pass of the two-pass scheme stores transposed, W rows at a time; beyond 512
        // points per row W gets too small for coalesced stores, and three passes are faster.
        // (ROCFFT_AMD_SPLIT_LEVELS=3 or 4 asks for that many passes where fewer would do: tests)
        const char* want_env = getenv("ROCFFT_AMD_SPLIT_LEVELS");
        const int   want     = want_env ? atoi(want_env) : 0;
        uint64_t n1 = 0, n0 = 0, n2 = 0;
        if(want < 3)
            split_two(n, esize, column, n1, n0, 512);
        if(n1 == 0)
        {
            if(want < 4)
                split_three(n, esize, column, n2, n1, n0);
            if(n2 == 0 && want < 3)
                split_two(n, esize, column, n1, n0);
            if(n2 == 0)
                n1 = want >= 3 ? 0 : n1;
        }
        std::vector<uint64_t> levels; // strided factors from the outermost in, then the row factor
        if(n2 != 0)
            levels = {n2, n1, n0};
        else if(n1 == 0)
        {
            // four passes: one more strided factor outside the three-pass scheme
            uint64_t a3, a2, a1, a0;
            split_four(n, esize, column, a3, a2, a1, a0);
            if(a3 != 0)
                levels = {a3, a2, a1, a0};
        }
        if(!levels.empty())
        {
            // Several passes, n = f0 f1 ... fL: pass i < L is a column FFT over the f_i samples that
            // lie R_i = f_{i+1} ... f_L apart inside each contiguous run of f_i R_i points, times
            // W_{f_i R_i}^{k_i r} (r the position inside the run of R_i); the last pass transforms the
            // contiguous runs of f_L points and stores result k_0 + f_0 (k_1 + f_1 (k_2 + ...)).
            // (Pass 0 reads the user's array, the others work in place in the scratch array.)
            const size_t L = levels.size() - 1;
            std::vector<uint64_t> R(L + 1, 1);
            for(size_t i = L; i-- > 0;)
                R[i] = R[i + 1] * levels[i + 1];
            b.need_tmp(lines * n);
            std::vector<int64_t> pk = packed_strides(n);
            for(size_t i = 0; i < L; ++i)
            {
                TileSpec s = base_spec();
                s.n        = (uint32_t)levels[i];
                s.t_is     = (int64_t)R[i] * (i == 0 ? t_is : 2);
                s.t_os     = (int64_t)R[i] * 2;
                s.src      = i == 0 ? src : tmp;
                s.dst      = tmp;
                s.others.push_back({(uint32_t)R[i], i == 0 ? t_is : 2, 2, true});
                for(size_t j = 0; j < i; ++j)
                    s.others.push_back({(uint32_t)levels[j], (int64_t)R[j] * 2, (int64_t)R[j] * 2, false});
                add_others(s, i == 0, false, pk);
                s.flags |= FFTK_F_TWIDDLE_STORE;
                const uint64_t span = levels[i] * R[i];
                s.ltw               = large_twiddles(span, b.precision, b.dry);
                s.ltw_shift         = large_twiddle_shift(span);
                static const char* names[3] = {"A (column fft over the outer factor + twiddle)",
                                               "B (column fft over the middle factor + twiddle)",
                                               "B2 (column fft over the inner strided factor + twiddle)"};
                s.note = dims_note((std::string(L == 2 ? "split3 " : "split4 ") + names[i]).c_str(), levels[i]);
                b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
            }
            {
                TileSpec s = base_spec();
                s.n        = (uint32_t)levels[L];
                s.t_is     = 2;
                uint64_t outer = 1; // f_0 ... f_{L-1}
                for(size_t j = 0; j < L; ++j)
                    outer *= levels[j];
                s.t_os = (int64_t)outer * t_os;
                s.src  = tmp;
                s.dst  = dst;
                uint64_t below = 1; // f_0 ... f_{j-1}
                std::vector<Axis> ax;
                for(size_t j = 0; j < L; ++j)
                {
                    ax.push_back({(uint32_t)levels[j], (int64_t)R[j] * 2, (int64_t)below * t_os, false});
                    below *= levels[j];
                }
                for(size_t j = L; j-- > 0;)
                    s.others.push_back(ax[j]);
                add_others(s, false, true, pk);
                if(ops.has_scale)
                {
                    s.flags |= FFTK_F_SCALE;
                    s.scale = ops.scale;
                }
                s.note = dims_note(L == 2 ? "split3 C (row fft, doubly transposed store)" : "split4 C (row fft, triply transposed store)",
                                   levels[L]);
                b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
            }
            return;
        }
        if(n1 == 0)
            fail("length too large for the two- and three-pass decompositions");
        // pass A: for every n0' an n1-point FFT over the stride-n0 samples, times W_n^{k1 n0'},
        // written to scratch at index k1*n0 + n0' of the dimension
        // pass B: for every k1 an n0-point FFT over n0', written to dst at k0*n1 + k1
        // (the reference's two-kernel large 1D, library/src/tree_node_1D.cpp:404-469)
        //
        // The scratch array keeps the axis order of the source: axes that run faster than this
        // dimension in the source (the columns of a strided dimension) stay innermost, so that
        // a tile of neighbouring columns is contiguous in the scratch array too; the other axes
        // are packed outside the dimension.
        std::vector<int64_t> pk(others.size(), 0);
        std::vector<size_t>  order(others.size());
        for(size_t i = 0; i < others.size(); ++i)
            order[i] = i;
        std::sort(order.begin(), order.end(),
                  [&](size_t x, size_t y) { return others[x].is < others[y].is; });
        int64_t inner = 1; // complex elements inside one step of this dimension
        for(size_t i : order)
            if(others[i].cnt > 1 && others[i].is < t_is)
            {
                pk[i] = 2 * inner;
                inner *= others[i].cnt;
            }
        // keep the pitch of the dimension off multiples of 2 KiB (HBM channel aliasing)
        int64_t innerP = inner;
        if(inner > 1 && ((size_t)inner * esize) % 2048 == 0)
            innerP += 16;
        const int64_t tS    = 2 * innerP; // scalar stride of the dimension in the scratch array
        int64_t       outer = (int64_t)n * tS;
        for(size_t i : order)
            if(!(others[i].cnt > 1 && others[i].is < t_is))
            {
                pk[i] = outer;
                outer *= others[i].cnt;
            }
        b.need_tmp((size_t)(outer / 2));
        TablePtr ltw = large_twiddles(n, b.precision, b.dry);
        {
            TileSpec s = base_spec();
            s.n        = (uint32_t)n1;
            s.t_is     = (int64_t)n0 * t_is;
            s.t_os     = (int64_t)n0 * tS;
            s.src      = src;
            s.dst      = tmp;
            s.others.push_back({(uint32_t)n0, t_is, tS, true});
            add_others(s, true, false, pk);
            s.flags |= FFTK_F_TWIDDLE_STORE;
            s.ltw       = ltw;
            s.ltw_shift = large_twiddle_shift(n);
            s.note      = dims_note("split A (column fft + twiddle)", n1);
            b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
        }
        {
            TileSpec s = base_spec();
            s.n        = (uint32_t)n0;
            s.t_is     = tS;
            s.t_os     = (int64_t)n1 * t_os;
            s.src      = tmp;
            s.dst      = dst;
            s.others.push_back({(uint32_t)n1, (int64_t)n0 * tS, t_os, false});
            add_others(s, false, true, pk);
            if(ops.has_scale)
            {
                s.flags |= FFTK_F_SCALE;
                s.scale = ops.scale;
            }
            s.note = dims_note(inner > 1 ? "split B (column fft, transposed store)" : "split B (row fft, transposed store)", n0);
            b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
        }
        return;
    }

    // Bluestein chirp-z (reference: library/src/tree_node_bluestein.cpp:27-285,
    // library/src/rtc_bluestein_gen.cpp:170-380).  The convolution length M is the
    // next power of two >= 2n-1 or a shorter length of compiled kernels; chirp and its spectrum are
    // plan-time tables.
    if(ops.store_op != FFTK_STORE_COMPLEX && ops.store_op != FFTK_STORE_REAL)
        fail("Bluestein cannot be combined with this real-transform step");
    if(ops.load_op == FFTK_LOAD_C2R_PRE)
        fail("Bluestein cannot be combined with this real-transform step");
    uint64_t N = n;
    uint64_t M = ceil_pow2(2 * N - 1);
    if(M >= (1ull << 31))
        fail("length too large");
    bool     conj_chirp = dir > 0;
    const uint64_t Mpow2 = M;
    auto one_kernel = [&](uint64_t m) {
        // the whole convolution in one workgroup when m fits; strided data must keep a wide tile
        bool ok = column ? column_kernel_length(m, esize) : single_kernel_length(m, esize);
        if(!ok && column && single_kernel_length(m, esize) && m <= 4096)
            ok = true;
        return ok;
    };
    // Any length >= 2n-1 serves; a power of two can be almost twice that.  A shorter length made
    // of compiled kernels is taken when it saves at least 30 % of the padded size (measured: no gain
    // at 27 %; the kernels of other lengths are somewhat slower than those of powers of two).
    uint64_t sM1 = 0, sM0 = 0; // factors of a shorter length for the three-kernel form
    if(g_use_fast && !getenv("ROCFFT_AMD_BLU_POW2"))
    {
        const uint64_t need = 2 * N - 1, lim = Mpow2 / 10 * 7;
        uint64_t       best = 0;
        for(uint64_t m = need; m < lim && m <= 16384; ++m)
            if(fast_kernel_exists(m, esize) && (one_kernel(m) || (!column && wide_kernel_length(m, esize))))
            {
                best = m;
                break;
            }
        if(best == 0 && !one_kernel(Mpow2) && !(!column && wide_kernel_length(Mpow2, esize)))
        {
            // m = m1 * m0: m0 the row factor (one convolution kernel per row), m1 the strided one
            const uint64_t lo0 = column ? 64 : 1024, lo1 = column ? 64 : 2;
            for(uint64_t m0 = 4096; m0 >= lo0; --m0)
            {
                if(!fast_kernel_exists(m0, esize) || !single_kernel_length(m0, esize))
                    continue;
                uint64_t m1 = std::max<uint64_t>(lo1, (need + m0 - 1) / m0);
                for(int step = 0; step < 64 && m1 * m0 < lim
                                  && !(fast_kernel_exists(m1, esize) && column_kernel_length(m1, esize));
                    ++step)
                    ++m1;
                if(!(fast_kernel_exists(m1, esize) && column_kernel_length(m1, esize)))
                    continue;
                if(m1 * m0 < lim && (best == 0 || m1 * m0 < best))
                {
                    best = m1 * m0;
                    sM1  = m1;
                    sM0  = m0;
                }
            }
        }
        if(best != 0)
            M = best;
    }
    bool one = sM1 == 0 && one_kernel(M);
    // single precision: the wide compiled kernels (up to M = 16384) still fit one workgroup
    bool wide_one = sM1 == 0 && !one && !column && wide_kernel_length(M, esize);
    // (checked before any table is computed: a chirp of 10^8 entries takes a minute)
    if(!one && !wide_one && (ops.load_op == FFTK_LOAD_HERM_EXPAND || ops.n_out))
        fail("odd-length real transforms of this size are not implemented");
    // rows of 4096 points in the three-kernel form, 8192 where that keeps the strided factor
    // within one kernel
    uint64_t row_len = 4096;
    if(!one && sM1 == 0 && !single_kernel_length(M / row_len, esize) && single_kernel_length(8192, esize))
        row_len = 8192;
    // Beyond row_len^2 points (2^26) the strided factor no longer fits one kernel either: three
    // levels, M = M2 * M1 * M0 (below).  ROCFFT_AMD_BLU3=<m1>,<m0> forces that form with these two
    // factors at any length they divide (tests, comparisons).
    uint64_t M2 = 0, f1 = 0, f0 = 0;
    {
        const char*        env = getenv("ROCFFT_AMD_BLU3");
        unsigned long long a = 0, c = 0;
        if(env && sscanf(env, "%llu,%llu", &a, &c) == 2 && a > 1 && c > 1 && Mpow2 % (a * c) == 0 && Mpow2 / (a * c) > 1)
        {
            M   = Mpow2;
            sM1 = sM0 = 0;
            one       = false;
            f1        = a;
            f0        = c;
            M2        = M / (a * c);
            wide_one  = false;
        }
    }
    // ... and well before that the strided passes of the two-level form, whose tiles hold whole
    // columns of M / 4096 points, are down to rows of 8 or 16 bytes.  Measured on MI355X, two
    // levels against three (single precision, one transform): M = 2^24 0.79 against 0.40 ms,
    // 2^25 2.10 against 0.83 ms, 2^26 2.85 against 1.62 ms (double precision 0.94 / 0.72, 2.46 / 1.38,
    // 4.35 / 2.61 ms); with two transforms M = 2^24 is a tie (0.76 ms both, double precision 1.16
    // against 1.31 ms) and below that two levels win (2^23 x 4: 0.62 against 0.73 ms).
    const bool long_columns = M / 4096 >= 8192 || (M / 4096 >= 4096 && lines == 1);
    if(M2 == 0 && !one && !wide_one && sM1 == 0 && (long_columns || !single_kernel_length(M / row_len, esize)))
    {
        // rows of 4096 points; the middle factor as long as a strided pass with full tile rows
        // takes (fewer launches of the row kernel), the rest to the outer factor
        f0 = 4096;
        for(f1 = 4096; f1 >= 64; f1 /= 2)
            if(column_kernel_length(f1, esize) && M / (f1 * f0) >= 2 && column_kernel_length(M / (f1 * f0), esize))
                break;
        if(f1 < 64)
            fail("Bluestein length too large");
        M2 = M / (f1 * f0);
    }
    if(M2 != 0
       && !(M2 >= 2 && column_kernel_length(M2, esize) && column_kernel_length(f1, esize) && single_kernel_length(f0, esize)))
        fail("Bluestein length too large");
    TablePtr chirp      = chirp_table(N, b.precision, b.dry);
    double   scale      = (1.0 / (double)M) * (ops.has_scale ? ops.scale : 1.0);
    uint32_t cflag      = conj_chirp ? FFTK_F_CHIRP_CONJ : 0;
    auto emit_one = [&]() {
        TablePtr bs = bluestein_spectrum(b, N, M, 0, 0, conj_chirp);
        TileSpec s  = base_spec();
        s.dir       = -1;
        s.n         = (uint32_t)M;
        s.t_is      = t_is;
        s.t_os      = t_os;
        s.src       = src;
        s.dst       = dst;
        add_others(s, true, true, {});
        s.load_op         = ops.load_op;
        s.store_op        = ops.store_op;
        s.src_real_scalar = ops.src_real_scalar;
        s.dst_real_scalar = ops.dst_real_scalar;
        s.n_in            = (uint32_t)N;
        s.n_out           = ops.n_out ? ops.n_out : (uint32_t)N;
        s.flags |= FFTK_F_CHIRP_LOAD | FFTK_F_CHIRP_STORE | FFTK_F_CONV | FFTK_F_SCALE | cflag;
        s.chirp    = chirp;
        s.blu_n    = (uint32_t)N;
        s.chirp_js = 1;
        s.chirp_qs = 0;
        s.convb    = bs;
        s.convb_qs = 0;
        s.scale    = scale;
        s.note     = dims_note("bluestein single kernel, M", M);
        b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
    };
    if(one)
    {
        emit_one();
        return;
    }
    if(wide_one)
    {
        const size_t mark = b.plan->passes.size();
        try
        {
            emit_one();
            return;
        }
        catch(const PlanError&)
        {
            b.plan->passes.resize(mark);
            if(M != Mpow2)
            {
                // this layout cannot use the wide kernel of the shorter length: back to the
                // power of two, in one kernel if that fits
                M     = Mpow2;
                scale = (1.0 / (double)M) * (ops.has_scale ? ops.scale : 1.0);
                if(one_kernel(M))
                {
                    emit_one();
                    return;
                }
            }
        }
    }
    if(ops.load_op == FFTK_LOAD_HERM_EXPAND || ops.n_out)
        fail("odd-length real transforms of this size are not implemented");
    if(M2 != 0)
    {
        // Three levels, M = M2 * M1 * M0, sample n = (n2 M1 + n1) M0 + n0, bin k = k2 + M2 (k1 + M1 k0):
        //   P1  chirp, pad, FFT over n2 (stride M1 M0), times W_M^{k2 (n1 M0 + n0)}            [like Z1]
        //   P2  in every block k2: FFT over n1 (stride M0), times W_{M1 M0}^{k1 n0}
        //   P3  one launch per block k2: every row (k2, k1) is transformed over n0, multiplied by
        //       its row of the chirp spectrum (kept in this order), transformed back and multiplied
        //       by conj W_M^{n0 (M2 k1 + k2)} -- the twiddle of the inverse over k1 and the part
        //       W_M^{k2 n0} of the twiddle of the inverse over k2, which does not depend on n1  [like Z2]
        //   P4  in every block k2: inverse FFT over k1, times conj W_{M2 M1}^{k2 n1} (the rest of it)
        //   P5  inverse FFT over k2, chirp, scale, first n outputs                              [like Z3]
        // The padded signals are M contiguous elements each (no row padding: the tile axis of P1 and
        // P5 runs over n1 and n0 together).
        const uint64_t M1 = f1, M0 = f0, R = M1 * M0;
        TablePtr bs = bluestein_spectrum(b, N, M, M1, M0, conj_chirp, M2);
        std::vector<int64_t> pk(others.size(), 0);
        int64_t              inner = 1;
        {
            std::vector<size_t> order(others.size());
            for(size_t i = 0; i < others.size(); ++i)
                order[i] = i;
            std::sort(order.begin(), order.end(), [&](size_t x, size_t y) { return others[x].is < others[y].is; });
            for(size_t i : order)
                if(column && others[i].cnt > 1 && others[i].is < t_is)
                {
                    pk[i] = 2 * inner;
                    inner *= others[i].cnt;
                }
            int64_t outer = (int64_t)M * 2 * inner;
            for(size_t i : order)
                if(pk[i] == 0)
                {
                    pk[i] = outer;
                    outer *= others[i].cnt;
                }
            b.need_blu((size_t)(outer / 2));
        }
        const int64_t qS = 2 * inner;
        {
            TileSpec s = base_spec();
            s.dir      = -1;
            s.n        = (uint32_t)M2;
            s.t_is     = (int64_t)R * t_is;
            s.t_os     = (int64_t)R * qS;
            s.src      = src;
            s.dst      = blu;
            s.others.push_back({(uint32_t)R, t_is, qS, true});
            add_others(s, true, false, pk);
            s.load_op         = ops.load_op;
            s.src_real_scalar = ops.src_real_scalar;
            s.flags |= FFTK_F_CHIRP_LOAD | FFTK_F_TWIDDLE_STORE | cflag;
            s.chirp     = chirp;
            s.blu_n     = (uint32_t)N;
            s.chirp_js  = (uint32_t)R;
            s.chirp_qs  = 1;
            s.ltw       = large_twiddles(M, b.precision, b.dry);
            s.ltw_shift = large_twiddle_shift(M);
            s.note      = dims_note("bluestein P1 (chirp, pad, column fft over the outer factor, twiddle)", M2);
            b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
        }
        {
            TileSpec s = base_spec();
            s.dir      = -1;
            s.n        = (uint32_t)M1;
            s.t_is = s.t_os = (int64_t)M0 * qS;
            s.src = s.dst = blu;
            s.others.push_back({(uint32_t)M0, qS, qS, true});
            s.others.push_back({(uint32_t)M2, (int64_t)R * qS, (int64_t)R * qS, false});
            add_others(s, false, false, pk);
            s.flags |= FFTK_F_TWIDDLE_STORE;
            s.ltw       = large_twiddles(R, b.precision, b.dry);
            s.ltw_shift = large_twiddle_shift(R);
            s.note      = dims_note("bluestein P2 (column fft over the middle factor, twiddle)", M1);
            b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
        }
        for(uint64_t k2 = 0; k2 < M2; ++k2)
        {
            TileSpec s = base_spec();
            s.dir      = -1;
            s.n        = (uint32_t)M0;
            s.t_is = s.t_os = qS;
            s.src = s.dst = blu;
            s.src_extra = s.dst_extra = (int64_t)(k2 * R) * qS;
            s.others.push_back({(uint32_t)M1, (int64_t)M0 * qS, (int64_t)M0 * qS, true});
            add_others(s, false, false, pk);
            s.flags |= FFTK_F_CONV | FFTK_F_TWIDDLE_STORE;
            s.convb     = bs;
            s.convb_qs  = (uint32_t)M0;
            s.convb_off = k2 * R;
            s.ltw       = large_twiddles(M, b.precision, b.dry);
            s.ltw_shift = large_twiddle_shift(M);
            s.ltw_qmul  = (uint32_t)M2;
            s.ltw_qadd  = (uint32_t)k2;
            s.note      = dims_note("bluestein P3 (rows of one block: fft, multiply, inverse fft, twiddle)", M0);
            b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
        }
        {
            TileSpec s = base_spec();
            s.dir      = +1;
            s.n        = (uint32_t)M1;
            s.t_is = s.t_os = (int64_t)M0 * qS;
            s.src = s.dst = blu;
            s.others.push_back({(uint32_t)M0, qS, qS, false});
            s.others.push_back({(uint32_t)M2, (int64_t)R * qS, (int64_t)R * qS, true});
            add_others(s, false, false, pk);
            s.flags |= FFTK_F_TWIDDLE_STORE;
            s.ltw       = large_twiddles(M2 * M1, b.precision, b.dry);
            s.ltw_shift = large_twiddle_shift(M2 * M1);
            s.note      = dims_note("bluestein P4 (inverse column fft over the middle factor, twiddle)", M1);
            b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
        }
        {
            TileSpec s = base_spec();
            s.dir      = +1;
            s.n        = (uint32_t)M2;
            s.t_is     = (int64_t)R * qS;
            s.t_os     = (int64_t)R * t_os;
            s.src      = blu;
            s.dst      = dst;
            s.others.push_back({(uint32_t)R, qS, t_os, true});
            add_others(s, false, true, pk);
            s.store_op        = ops.store_op;
            s.dst_real_scalar = ops.dst_real_scalar;
            s.flags |= FFTK_F_CHIRP_STORE | FFTK_F_SCALE | cflag;
            s.chirp    = chirp;
            s.blu_n    = (uint32_t)N;
            s.chirp_js = (uint32_t)R;
            s.chirp_qs = 1;
            s.scale    = scale;
            s.note     = dims_note("bluestein P5 (inverse column fft over the outer factor, chirp, scale)", M2);
            b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
        }
        return;
    }
    // M = M1*M0: rows of length M0 are transformed, multiplied and transformed back by
    // one kernel, so that kernel gets the long factor; the strided passes get M1
    uint64_t M0 = row_len, M1 = M / M0;
    if(sM1 != 0)
    {
        M1 = sM1;
        M0 = sM0;
    }
    else
    {
        // short strided passes make tiny workgroups: keep at least `floor` points in them
        static const char* env   = getenv("ROCFFT_AMD_BLU_M1");
        const uint64_t     floor = env ? (uint64_t)atoi(env) : (column ? 64 : 1);
        if(M1 < floor && M / floor >= 64)
        {
            M1 = floor;
            M0 = M / M1;
        }
    }
    while(M1 > 1 && !single_kernel_length(M1, esize))
        fail("Bluestein length too large");
    if(M1 < 2)
        fail("internal: Bluestein split of a short length");
    TablePtr bs  = bluestein_spectrum(b, N, M, M1, M0, conj_chirp);
    TablePtr ltw = large_twiddles(M, b.precision, b.dry);
    // rows of the padded signals get a pitch that is not a power of two, so that the strided
    // column passes do not hammer one HBM channel
    const int64_t rowp = (int64_t)M0 + 16; // complex elements
    // The padded signals keep the axis order of the source, like the scratch array of the
    // split: axes that run faster than this dimension (the columns of a strided dimension)
    // stay innermost, so that a tile of neighbouring columns is contiguous there as well and
    // all three passes are column passes over it; the other axes are packed outside.
    std::vector<int64_t> pk(others.size(), 0);
    int64_t              inner = 1;
    {
        std::vector<size_t> order(others.size());
        for(size_t i = 0; i < others.size(); ++i)
            order[i] = i;
        std::sort(order.begin(), order.end(),
                  [&](size_t x, size_t y) { return others[x].is < others[y].is; });
        for(size_t i : order)
            if(column && others[i].cnt > 1 && others[i].is < t_is)
            {
                pk[i] = 2 * inner;
                inner *= others[i].cnt;
            }
        int64_t outer = (int64_t)M1 * rowp * 2 * inner;
        for(size_t i : order)
            if(pk[i] == 0)
            {
                pk[i] = outer;
                outer *= others[i].cnt;
            }
        b.need_blu((size_t)(outer / 2));
    }
    const int64_t qS = 2 * inner; // scalar stride of one step along a padded signal
    {
        // Z1: chirp multiply + zero pad fused into the load of the column FFT over n1
        TileSpec s = base_spec();
        s.dir      = -1;
        s.n        = (uint32_t)M1;
        s.t_is     = (int64_t)M0 * t_is;
        s.t_os     = rowp * qS;
        s.src      = src;
        s.dst      = blu;
        s.others.push_back({(uint32_t)M0, t_is, qS, true});
        add_others(s, true, false, pk);
        s.load_op         = ops.load_op;
        s.src_real_scalar = ops.src_real_scalar;
        s.flags |= FFTK_F_CHIRP_LOAD | FFTK_F_TWIDDLE_STORE | cflag;
        s.chirp     = chirp;
        s.blu_n     = (uint32_t)N;
        s.chirp_js  = (uint32_t)M0;
        s.chirp_qs  = 1;
        s.ltw       = ltw;
        s.ltw_shift = large_twiddle_shift(M);
        s.note      = dims_note("bluestein Z1 (chirp, pad, column fft, twiddle)", M1);
        b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
    }
    {
        // Z2: row FFT, multiply by the chirp spectrum, inverse row FFT, conjugate twiddle
        TileSpec s = base_spec();
        s.dir      = -1;
        s.n        = (uint32_t)M0;
        s.t_is = s.t_os = qS;
        s.src = s.dst = blu;
        s.others.push_back({(uint32_t)M1, rowp * qS, rowp * qS, true});
        add_others(s, false, false, pk);
        s.flags |= FFTK_F_CONV | FFTK_F_TWIDDLE_STORE;
        s.convb     = bs;
        s.convb_qs  = (uint32_t)M0;
        s.ltw       = ltw;
        s.ltw_shift = large_twiddle_shift(M);
        s.note      = dims_note("bluestein Z2 (row fft, multiply, inverse row fft, twiddle)", M0);
        b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
    }
    {
        // Z3: inverse column FFT, multiply by the chirp, scale by 1/M, keep n outputs
        TileSpec s = base_spec();
        s.dir      = +1;
        s.n        = (uint32_t)M1;
        s.t_is     = rowp * qS;
        s.t_os     = (int64_t)M0 * t_os;
        s.src      = blu;
        s.dst      = dst;
        s.others.push_back({(uint32_t)M0, qS, t_os, true});
        add_others(s, false, true, pk);
        s.store_op        = ops.store_op;
        s.dst_real_scalar = ops.dst_real_scalar;
        s.flags |= FFTK_F_CHIRP_STORE | FFTK_F_SCALE | cflag;
        s.chirp    = chirp;
        s.blu_n    = (uint32_t)N;
        s.chirp_js = (uint32_t)M0;
        s.chirp_qs = 1;
        s.scale    = scale;
        s.note     = dims_note("bluestein Z3 (inverse column fft, chirp, scale)", M1);
        b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
    }
}

// FFT_M of the wrapped chirp, computed on the GPU in double precision with this
// library's own passes and narrowed to the plan precision.  For a split M the
// result is kept in the order the convolution kernel meets it: [k1*M0 + k0].
static TablePtr bluestein_spectrum(Builder& b, uint64_t N, uint64_t M, uint64_t M1, uint64_t M0,
                                   bool conj_chirp, uint64_t M2)
{
    std::ostringstream key;
    key << "bspec_" << N << "_" << M << "_" << M2 << "_" << M1 << "_" << M0 << (conj_chirp ? "c" : "f");
    int dev = 0;
    if(!b.dry)
        fftrt_device_info(&dev, nullptr, nullptr, nullptr, 0);
    key << "/p" << b.precision << "/d" << dev << (b.dry ? "/dry" : "");
    {
        std::lock_guard<std::mutex> lock(g_cache_mutex);
        auto                        it = g_cache.find(key.str());
        if(it != g_cache.end())
            if(TablePtr t = it->second.lock())
                return t;
    }
    TablePtr out(new DeviceTable);
    out->bytes = M * (b.precision ? 16 : 8);
    if(!b.dry)
    {
        std::vector<double> w(2 * M, 0.0);
        host_parallel(N, [&](uint64_t first, uint64_t last) {
            for(uint64_t m = first; m < last; ++m)
            {
                long double c, s;
                chirp_value(m, N, c, s);
                if(conj_chirp)
                    s = -s;
                w[2 * m]     = (double)c;
                w[2 * m + 1] = (double)s;
                if(m)
                {
                    w[2 * (M - m)]     = (double)c;
                    w[2 * (M - m) + 1] = (double)s;
                }
            }
        });
        void* dbuf = nullptr;
        if(fftrt_malloc(&dbuf, 2 * M * sizeof(double)) != 0)
            fail("device allocation failed");
        std::shared_ptr<void> guard(dbuf, [](void* p) { fftrt_free(p); });
        if(fftrt_upload(dbuf, w.data(), 2 * M * sizeof(double)) != 0)
            fail("upload failed");
        ExecPlan sub;
        sub.precision  = 1;
        sub.elem_bytes = 16;
        Builder sb{&sub, 1, false, 16};
        IoRef   io;
        io.buf = BUF_IN;
        DimOps none;
        if(M1 == 0)
            emit_dim(sb, M, 2, 2, {}, io, io, -1, none);
        else if(M2 > 1)
        {
            // three levels: the forward passes of the convolution itself, order [k2][k1][k0]
            const uint64_t R = M1 * M0;
            TileSpec       a;
            a.dir  = -1;
            a.n    = (uint32_t)M2;
            a.t_is = a.t_os = (int64_t)R * 2;
            a.src = a.dst = io;
            a.others.push_back({(uint32_t)R, 2, 2, true});
            a.flags |= FFTK_F_TWIDDLE_STORE;
            a.ltw       = large_twiddles(M, 1, false);
            a.ltw_shift = large_twiddle_shift(M);
            sub.passes.push_back(make_tile_pass(a, 1, false));
            TileSpec c;
            c.dir  = -1;
            c.n    = (uint32_t)M1;
            c.t_is = c.t_os = (int64_t)M0 * 2;
            c.src = c.dst = io;
            c.others.push_back({(uint32_t)M0, 2, 2, true});
            c.others.push_back({(uint32_t)M2, (int64_t)R * 2, (int64_t)R * 2, false});
            c.flags |= FFTK_F_TWIDDLE_STORE;
            c.ltw       = large_twiddles(R, 1, false);
            c.ltw_shift = large_twiddle_shift(R);
            sub.passes.push_back(make_tile_pass(c, 1, false));
            TileSpec r;
            r.dir  = -1;
            r.n    = (uint32_t)M0;
            r.t_is = r.t_os = 2;
            r.src = r.dst = io;
            r.others.push_back({(uint32_t)(M2 * M1), (int64_t)M0 * 2, (int64_t)M0 * 2, false});
            sub.passes.push_back(make_tile_pass(r, 1, false));
        }
        else
        {
            TablePtr ltw = large_twiddles(M, 1, false);
            TileSpec a;
            a.dir  = -1;
            a.n    = (uint32_t)M1;
            a.t_is = a.t_os = (int64_t)M0 * 2;
            a.src = a.dst = io;
            a.others.push_back({(uint32_t)M0, 2, 2, true});
            a.flags |= FFTK_F_TWIDDLE_STORE;
            a.ltw       = ltw;
            a.ltw_shift = large_twiddle_shift(M);
            sub.passes.push_back(make_tile_pass(a, 1, false));
            TileSpec r;
            r.dir  = -1;
            r.n    = (uint32_t)M0;
            r.t_is = r.t_os = 2;
            r.src = r.dst = io;
            r.others.push_back({(uint32_t)M1, (int64_t)M0 * 2, (int64_t)M0 * 2, false});
            sub.passes.push_back(make_tile_pass(r, 1, false));
        }
        void* bufs[2] = {dbuf, nullptr};
        void* sub_work = nullptr;
        if(sub.work_bytes() && fftrt_malloc(&sub_work, sub.work_bytes()) != 0)
            fail("device allocation failed");
        std::shared_ptr<void> work_guard(sub_work, [](void* p) {
            if(p)
                fftrt_free(p);
        });
        if(run_exec_plan(sub, bufs, bufs, sub_work, nullptr) != rocfft_status_success)
            fail("computing the Bluestein chirp spectrum failed");
        if(fftrt_stream_sync(nullptr) != 0)
            fail("computing the Bluestein chirp spectrum failed");
        if(fftrt_download(w.data(), dbuf, 2 * M * sizeof(double)) != 0)
            fail("download failed");
        if(fftrt_malloc(&out->dptr, out->bytes) != 0)
            fail("device allocation failed");
        int rc;
        if(b.precision)
            rc = fftrt_upload(out->dptr, w.data(), out->bytes);
        else
        {
            std::vector<float> f(2 * M);
            for(size_t i = 0; i < 2 * M; ++i)
                f[i] = (float)w[i];
            rc = fftrt_upload(out->dptr, f.data(), out->bytes);
        }
        if(rc != 0)
            fail("upload failed");
    }
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    g_cache[key.str()] = out;
    return out;
}

// The one-workgroup 32768-point kernel (big_kernels.hip): single precision, unit stride
// along the transform on both sides, interleaved data, at most three line dimensions.
// mode 0: complex (src/dst complex interleaved), 1: real forward (src real pairs, dst
// Hermitian), 2: real inverse (src Hermitian, dst real pairs).
static bool big_eligible(const Builder& b, uint64_t n, int64_t t_is, int64_t t_os,
                         const std::vector<Other>& others, const IoRef& src, const IoRef& dst)
{
    if(!g_use_fast || getenv("ROCFFT_AMD_NO_BIG") || b.precision != 0 || n != 32768)
        return false;
    if(!fftrt_has_big32k())
        return false;
    if(src.planar || dst.planar || src.im_delta != 1 || dst.im_delta != 1 || t_is != 2 || t_os != 2)
        return false;
    if((src.off0 & 1) || (dst.off0 & 1))
        return false;
    size_t cnt = 0;
    for(const Other& o : others)
        if(o.cnt > 1)
        {
            ++cnt;
            if((o.is & 1) || (o.os & 1))
                return false;
        }
    return cnt <= 3;
}

static void emit_big(Builder& b, uint32_t mode, const std::vector<Other>& others, const IoRef& src,
                     const IoRef& dst, int dir, double scale, bool has_scale)
{
    PassRec rec;
    rec.kind = PASS_BIG;
    memset(&rec.kp, 0, sizeof(rec.kp));
    memset(&rec.rp, 0, sizeof(rec.rp));
    fftk_big_params& q = rec.bp;
    memset(&q, 0, sizeof(q));
    double lines = 1;
    int    i     = 0;
    for(int d = 0; d < 3; ++d)
        q.lines[d] = 1;
    for(const Other& o : others)
        if(o.cnt > 1)
        {
            q.lines[i]    = o.cnt;
            q.in_line[i]  = o.is;
            q.out_line[i] = o.os;
            lines *= o.cnt;
            ++i;
        }
    q.mode      = mode;
    q.dir       = dir;
    q.scale     = scale;
    q.use_scale = has_scale ? 1 : 0;
    uint32_t twoff[FFTK_MAX_PASSES];
    TablePtr tw = stacked_twiddles({32, 32, 32}, 0, b.dry, twoff);
    TablePtr ha = cached_table("bigA", 0, b.dry, [](HostTable& h) {
        for(uint64_t t = 0; t < 1024; ++t)
        {
            long double c, s;
            unit_root(t, 65536, c, s);
            h.push(c, s);
        }
    });
    TablePtr hb = cached_table("bigB", 0, b.dry, [](HostTable& h) {
        for(uint64_t k = 0; k < 32; ++k)
        {
            long double c, s;
            unit_root(k, 64, c, s);
            h.push(c, s);
        }
    });
    q.tw     = tw->dptr;
    q.half_a = ha->dptr;
    q.half_b = hb->dptr;
    rec.tables.push_back(tw);
    rec.tables.push_back(ha);
    rec.tables.push_back(hb);
    rec.src  = src;
    rec.dst  = dst;
    rec.grid = (uint32_t)lines;
    rec.lds  = 0;
    static const char* names[3] = {"one-workgroup fft n=32768", "one-workgroup real forward n=65536",
                                   "one-workgroup real inverse n=65536"};
    rec.note     = names[mode];
    rec.bytes_rw = lines * (mode == 0 ? 2.0 * 32768 * 8 : (65536.0 * 4 + 32769.0 * 8));
    b.plan->passes.push_back(rec);
}

// Dimensions 0 and 1 of a complex transform in one kernel, when both are small powers of two
// and every 2D slice is a contiguous block on both sides.  Returns false (nothing emitted) when
// the runtime has no such kernel for these sizes or the layout does not fit.
static const bool g_use_2d = !getenv("ROCFFT_AMD_NO_2D");

// mode 0: complex; 1: real forward (in = the real rows seen as pairs, out = Hermitian rows);
// 2: real inverse (in = Hermitian rows, out = real pairs).  len[0] is the transform length of
// dimension 0 (the real length for modes 1 and 2, which must be even).
static bool emit_fused_2d(Builder& b, int mode, const size_t* len, size_t rank, size_t batch, const View& in,
                          const View& out, int dir, double scale, bool has_scale)
{
    if(!g_use_fast || !g_use_2d || rank < 2)
        return false;
    if(mode != 0 && (len[0] % 2 || len[0] < 8))
        return false;
    const size_t nA = mode ? len[0] / 2 : len[0]; // complex points per row that the row phase transforms
    const size_t nB = len[1], esize = b.esize;
    const size_t rowlen = mode ? nA + 1 : nA;     // elements per row of the LDS tile
    uint32_t     ra[4], rb[4], nfa = 0, nfb = 0, tpta = 0, tptb = 0, pitch = 0;
    if(nA > 64 || nB > 64)
        return false;
    int have = mode ? fftrt_fast2d_real_info((uint32_t)nA, (uint32_t)nB, ra, &nfa, rb, &nfb, &tpta, &tptb, &pitch)
                    : fftrt_fast2d_info((uint32_t)nA, (uint32_t)nB, ra, &nfa, rb, &nfb, &tpta, &tptb, &pitch);
    if(!have)
        return false;
    auto plain = [](const IoRef& io) { return !io.planar && io.im_delta == 1 && io.off0 % 2 == 0; };
    if(!plain(in.io) || !plain(out.io))
        return false;
    // unit stride along dimension 0, whole complex elements between rows
    if(in.stride[0] != 2 || out.stride[0] != 2 || in.stride[1] <= 0 || out.stride[1] <= 0 || in.stride[1] % 2
       || out.stride[1] % 2 || in.stride[1] / 2 >= (1ll << 24) || out.stride[1] / 2 >= (1ll << 24))
        return false;
    // the axes that enumerate the 2D slices: dimension 2 (if any) and the batch
    std::vector<Axis> ax;
    if(rank == 3 && len[2] > 1)
        ax.push_back({(uint32_t)len[2], in.stride[2], out.stride[2], false});
    if(batch > 1)
        ax.push_back({(uint32_t)batch, in.stride[3], out.stride[3], false});
    for(const Axis& a : ax)
        if(a.is % 2 || a.os % 2 || a.is <= 0 || a.os <= 0)
            return false;
    // merge when the batch continues dimension 2
    if(ax.size() == 2 && ax[0].is * (int64_t)ax[0].cnt == ax[1].is && ax[0].os * (int64_t)ax[0].cnt == ax[1].os
       && (uint64_t)ax[0].cnt * ax[1].cnt < (1ull << 31))
    {
        ax[0].cnt *= ax[1].cnt;
        ax.pop_back();
    }
    Axis tile = {1, in.stride[1] * (int64_t)nB, out.stride[1] * (int64_t)nB, false};
    if(!ax.empty())
    {
        size_t t = (ax.size() == 2 && ax[1].is < ax[0].is) ? 1 : 0;
        tile     = ax[t];
        ax.erase(ax.begin() + (long)t);
    }
    const size_t tp       = nB * (size_t)pitch; // LDS elements per transform
    const size_t max_elem = esize == 8 ? 4096 : 2048;
    uint32_t     tpx      = (uint32_t)std::max(nB * tpta, rowlen * tptb);
    uint32_t     K        = floor_pow2(std::max<size_t>(1, max_elem / (rowlen * nB)));
    K                     = std::min(K, floor_pow2(std::max<uint32_t>(1, 256 / tpx)));
    K                     = std::min(K, ceil_pow2(tile.cnt));
    if(K * tpx > 512 || K * tp * esize > 64 * 1024)
        return false;
    if((uint64_t)K * (uint64_t)(tile.is / 2) >= (1ull << 31) || (uint64_t)K * (uint64_t)(tile.os / 2) >= (1ull << 31))
        return false;

    PassRec rec;
    rec.kind = PASS_2D;
    rec.src  = in.io;
    rec.dst  = out.io;
    fftk_params& k = rec.kp;
    memset(&k, 0, sizeof(k));
    k.n  = (uint32_t)nA;
    k.n2 = (uint32_t)nB;
    k.nf = nfa;
    std::vector<uint32_t> va(ra, ra + nfa), vb(rb, rb + nfb);
    for(uint32_t i = 0; i < nfa; ++i)
        k.radix[i] = ra[i];
    uint32_t twoff_a[FFTK_MAX_PASSES], twoff_b[FFTK_MAX_PASSES];
    TablePtr twa = stacked_twiddles(va, b.precision, b.dry, twoff_a);
    TablePtr twb = stacked_twiddles(vb, b.precision, b.dry, twoff_b);
    k.tw         = twa->dptr;
    k.tw2        = twb->dptr;
    rec.tables.push_back(twa);
    rec.tables.push_back(twb);
    if(mode)
    {
        TablePtr htw = half_twiddles(nA, b.precision, b.dry);
        k.half_tw    = htw->dptr;
        rec.tables.push_back(htw);
    }
    k.T        = tpta;
    k.W        = K;
    k.wshift   = log2u(K);
    k.pitch    = pitch;
    k.padshift = PADSHIFT;
    k.tile_cnt = tile.cnt;
    k.w_is     = tile.is;
    k.w_os     = tile.os;
    k.w_is_c   = (uint32_t)(tile.is / 2);
    k.w_os_c   = (uint32_t)(tile.os / 2);
    k.t_is     = in.stride[1];
    k.t_os     = out.stride[1];
    k.t_is_c   = (uint32_t)(in.stride[1] / 2);  // complex elements between rows
    k.t_os_c   = (uint32_t)(out.stride[1] / 2);
    for(int i = 0; i < 3; ++i)
    {
        k.oc[i]   = 1;
        k.o_is[i] = k.o_os[i] = 0;
    }
    for(size_t i = 0; i < ax.size(); ++i)
    {
        k.oc[i]   = ax[i].cnt;
        k.o_is[i] = ax[i].is;
        k.o_os[i] = ax[i].os;
    }
    k.nthreads    = (K * tpx + 63) / 64 * 64;
    uint64_t grid = (uint64_t)((tile.cnt + K - 1) / K) * k.oc[0] * k.oc[1] * k.oc[2];
    if(grid == 0 || grid >= (1ull << 31))
        return false;
    rec.grid = k.grid = (uint32_t)grid;
    rec.lds           = K * tp * esize;
    k.fast            = 1;
    k.dir             = dir;
    k.load_op         = mode == 2 ? FFTK_LOAD_C2R_PRE : FFTK_LOAD_COMPLEX;
    k.store_op        = mode == 1 ? FFTK_STORE_R2C_POST : FFTK_STORE_COMPLEX;
    k.n_in = k.n_out = (uint32_t)nA;
    if(has_scale)
    {
        k.flags |= FFTK_F_SCALE;
        k.scale = scale;
    }
    rec.vec_ok         = true;
    const double lines = (double)tile.cnt * k.oc[0] * k.oc[1] * k.oc[2];
    rec.bytes_rw       = (mode ? (double)(nA + rowlen) : 2.0 * (double)nA) * (double)nB * lines * (double)esize;
    std::ostringstream note;
    note << (mode == 1 ? "2D real forward fft " : mode == 2 ? "2D real inverse fft " : "2D fft ") << len[0] << "x" << nB
         << " in one workgroup";
    rec.note = note.str();
    b.plan->passes.push_back(rec);
    return true;
}

// element-wise copy of `cnt` elements per row between two array kinds (fftk_copy_params)
static void emit_copy(Builder& b, uint32_t cnt, const std::vector<Other>& rows, int64_t s_s, const IoRef& src,
                      int64_t d_s, const IoRef& dst, const fftk_copy_params& proto, const char* what)
{
    if(rows.size() > 3)
        fail("too many dimensions");
    PassRec rec;
    rec.kind = PASS_COPY;
    memset(&rec.kp, 0, sizeof(rec.kp));
    fftk_copy_params& c = rec.cp;
    c                   = proto;
    c.cnt               = cnt;
    c.rows0 = c.rows1 = c.rows2 = 1;
    uint32_t* rc[3]             = {&c.rows0, &c.rows1, &c.rows2};
    int64_t*  ss[3]             = {&c.s_r0, &c.s_r1, &c.s_r2};
    int64_t*  ds[3]             = {&c.d_r0, &c.d_r1, &c.d_r2};
    double    rowsn             = 1;
    for(size_t i = 0; i < rows.size(); ++i)
    {
        *rc[i] = rows[i].cnt;
        *ss[i] = rows[i].is;
        *ds[i] = rows[i].os;
        rowsn *= rows[i].cnt;
    }
    c.s_s   = s_s;
    c.d_s   = d_s;
    rec.src = src;
    rec.dst = dst;
    rec.note     = dims_note(what, cnt);
    rec.bytes_rw = rowsn * cnt * (double)((c.src_real ? 1 : 2) + (c.dst_real ? 1 : 2)) * (b.precision ? 8 : 4);
    b.plan->passes.push_back(rec);
}

// Odd-length real transform whose length needs more than one kernel: the rows are copied
// into a complex scratch array (the reference's CS_REAL_TRANSFORM_USING_CMPLX scheme,
// library/src/tree_node_real.cpp:115-206), transformed there as complex data, and copied out.
// `lines`: the other dimensions and the batch, is = stride on the real side, os = stride on
// the Hermitian side.
static void emit_dim(Builder& b, uint64_t n, int64_t t_is, int64_t t_os, const std::vector<Other>& others,
                     const IoRef& src, const IoRef& dst, int dir, const DimOps& ops);

static void emit_odd_real_via_complex(Builder& b, bool forward, uint64_t n, const std::vector<Other>& lines,
                                      int64_t real_stride, const IoRef& real_io, int64_t herm_stride,
                                      const IoRef& herm_io, double scale, bool has_scale)
{
    const uint64_t h = n / 2 + 1;
    // packed complex rows in the scratch region
    std::vector<Other> packed, in_rows, out_rows;
    int64_t            st = 2 * (int64_t)n;
    uint64_t           total = n;
    for(const Other& o : lines)
    {
        packed.push_back({o.cnt, st, st});
        in_rows.push_back({o.cnt, forward ? o.is : o.os, st});
        out_rows.push_back({o.cnt, st, forward ? o.os : o.is});
        st *= o.cnt;
        total *= o.cnt;
    }
    b.need_cpx(total);
    IoRef cpx;
    cpx.buf = BUF_CPX;
    fftk_copy_params proto;
    memset(&proto, 0, sizeof(proto));
    if(forward)
    {
        proto.src_real = 1;
        emit_copy(b, (uint32_t)n, in_rows, real_stride, real_io, 2, cpx, proto, "real rows to complex scratch");
        emit_dim(b, n, 2, 2, packed, cpx, cpx, -1, DimOps());
        memset(&proto, 0, sizeof(proto));
        proto.scale     = scale;
        proto.use_scale = has_scale ? 1 : 0;
        emit_copy(b, (uint32_t)h, out_rows, 2, cpx, herm_stride, herm_io, proto, "first bins to Hermitian rows");
    }
    else
    {
        proto.mirror_from = (uint32_t)h;
        proto.mirror_n    = (uint32_t)n;
        proto.zero_im0    = 1;
        emit_copy(b, (uint32_t)n, in_rows, herm_stride, herm_io, 2, cpx, proto,
                  "Hermitian rows to full complex scratch");
        emit_dim(b, n, 2, 2, packed, cpx, cpx, +1, DimOps());
        memset(&proto, 0, sizeof(proto));
        proto.dst_real  = 1;
        proto.scale     = scale;
        proto.use_scale = has_scale ? 1 : 0;
        emit_copy(b, (uint32_t)n, out_rows, 2, cpx, real_stride, real_io, proto, "real parts to real rows");
    }
}

// standalone even-length post/pre pass over natural-order rows
static void emit_real_step(Builder& b, PassKind kind, uint64_t half, const std::vector<Other>& rows,
                           int64_t z_s, const IoRef& z, int64_t h_s, const IoRef& h, double scale,
                           bool has_scale)
{
    // rows: is = stride on the complex (z) side, os = stride on the Hermitian (h) side
    if(rows.size() > 3)
        fail("too many dimensions");
    PassRec rec;
    rec.kind = kind;
    memset(&rec.kp, 0, sizeof(rec.kp));
    fftk_real_params& r = rec.rp;
    memset(&r, 0, sizeof(r));
    r.half  = (uint32_t)half;
    r.rows0 = r.rows1 = r.rows2 = 1;
    uint32_t* cnt[3]            = {&r.rows0, &r.rows1, &r.rows2};
    int64_t*  zs[3]             = {&r.z_r0, &r.z_r1, &r.z_r2};
    int64_t*  hs[3]             = {&r.h_r0, &r.h_r1, &r.h_r2};
    for(size_t i = 0; i < rows.size(); ++i)
    {
        *cnt[i] = rows[i].cnt;
        *zs[i]  = rows[i].is;
        *hs[i]  = rows[i].os;
    }
    r.z_s         = z_s;
    r.h_s         = h_s;
    r.scale       = scale;
    r.use_scale   = has_scale ? 1 : 0;
    TablePtr tw   = half_twiddles(half, b.precision, b.dry);
    r.half_tw     = tw->dptr;
    rec.tables.push_back(tw);
    if(kind == PASS_REAL_POST)
    {
        rec.src = z;
        rec.dst = h;
    }
    else
    {
        rec.src = h;
        rec.dst = z;
    }
    {
        double rowsn = 1;
        for(const Other& o : rows)
            rowsn *= o.cnt;
        rec.bytes_rw = rowsn * (2.0 * half + 1) * 2 * (b.precision ? 8 : 4);
    }
    rec.note = dims_note(kind == PASS_REAL_POST ? "real post-process" : "real pre-process", 2 * half);
    b.plan->passes.push_back(rec);
}

// A single-pass dimension d followed by a long strided dimension e = d+1 (a "column"
// dimension too long for one column tile, e.g. the second dimension of a 4096 x 4096
// transform).  The pass over d writes its rows into the work buffer in permuted order (row
// n1*n0 + n0' of dimension e goes to slot n0'*n1 + n1): pass A of the split then reads n1
// consecutive rows where the plain split reads rows n0 apart, and pass B reads the strided rows
// before writing the user's output.  Measured on MI355X against the plain split of the same
// lengths: 4096 x 4096 x 8 single precision 1.23 against 1.28 ms, the other shapes tried
// (2048^2 ... 8192^2, 512 x 16384, both precisions) within 3 % either way.
static bool emit_dims_staged(Builder& b, const size_t* len, size_t rank, size_t batch, size_t d,
                             const View& src, const View& out, int dir, const DimOps& last_ops)
{
    const size_t e = d + 1;
    if(e >= rank || getenv("ROCFFT_AMD_NO_STAGED"))
        return false;
    const size_t   esize = b.esize;
    const uint64_t n     = len[e];
    // dimension e must be strided on both sides and too long for one column tile
    bool column = false;
    for(size_t i = 0; i < rank; ++i)
        if(i != e && len[i] > 1 && (src.stride[i] < src.stride[e] || out.stride[i] < out.stride[e]))
            column = true;
    if(!column || !smooth(n) || plain_dim_is_single(n, true, esize, src.stride[e], out.stride[e]))
        return false;
    // the tiles of the staged passes are as wide as the rows below dimension e are long; with
    // short rows the plain split is faster (its pass A merges the rows into wider tiles)
    uint64_t below = 1;
    for(size_t i = 0; i < e; ++i)
        below *= len[i];
    if(below < 64)
        return false;
    uint64_t n1, n0;
    split_length(n, esize, true, n1, n0);
    if(n1 == 0)
        return false;
    // dimension d must be one plain tile pass
    bool d_column = false;
    for(size_t i = 0; i < rank; ++i)
        if(i != d && len[i] > 1 && (src.stride[i] < src.stride[d]))
            d_column = true;
    int64_t d_packed = 2; // stride of dimension d in the packed intermediate array
    for(size_t i = 0; i < d; ++i)
        d_packed *= (int64_t)len[i];
    if(!plain_dim_is_single(len[d], d_column, esize, src.stride[d], d_packed))
        return false;
    if(src.io.planar || out.io.planar)
        return false;

    // packed layout of the intermediate array in TMP (scalars)
    int64_t tstride[4];
    int64_t run = 2;
    for(size_t i = 0; i < e; ++i)
    {
        tstride[i] = run;
        run *= (int64_t)len[i];
    }
    // Pitch between the rows of dimension e: the row itself, no padding.  Sum of pass A and B over
    // paddings of 0 / 128 / 256 / 512 / 1024 bytes, MI355X: 4096 x 4096 x 8 single 0.803 / 0.821 /
    // 0.882 / 0.808 / 0.827 ms; 8192 x 8192 single 0.406 / 0.408 / 0.411 / 0.517 / 0.411;
    // 4096 x 4096 x 4 double 0.846 / 0.831 / 0.824 / 0.970 / 0.840; 8192 x 8192 double 0.807 / 0.806 /
    // 0.804 / 0.820 / 1.092: every padding tried is the slow one for some shape (rows that come to
    // lie 2^k + 32 KiB apart), the power-of-two pitch for none of fourteen.
    // ROCFFT_AMD_STAGE_PAD sets the padding in scalars (comparisons).
    static const char* pad_env = getenv("ROCFFT_AMD_STAGE_PAD");
    const int64_t      rowS    = run + (pad_env ? atol(pad_env) : 0);
    const int64_t      s_n1 = rowS, s_n0 = (int64_t)n1 * rowS;
    run                = (int64_t)n0 * s_n0;
    for(size_t i = e + 1; i < rank; ++i)
    {
        tstride[i] = run;
        run *= (int64_t)len[i];
    }
    const int64_t tbatch = run;
    b.need_tmp((size_t)(tbatch / 2) * batch);
    IoRef tmp;
    tmp.buf = BUF_TMP;

    // pass over d: src -> TMP, dimension e split into (n0', n1') with permuted strides
    {
        std::vector<Other> oth;
        for(size_t i = 0; i < rank; ++i)
        {
            if(i == d)
                continue;
            if(i == e)
            {
                oth.push_back({(uint32_t)n0, src.stride[e], s_n0});
                oth.push_back({(uint32_t)n1, (int64_t)n0 * src.stride[e], s_n1});
            }
            else
                oth.push_back({(uint32_t)len[i], src.stride[i], tstride[i]});
        }
        oth.push_back({(uint32_t)batch, src.stride[3], tbatch});
        emit_dim(b, len[d], src.stride[d], tstride[d], oth, src.io, tmp, dir, DimOps());
    }
    TablePtr ltw = large_twiddles(n, b.precision, b.dry);
    // pass A: n1-point FFT over consecutive rows of TMP, in place, times W_n^{k1 n0'}
    {
        TileSpec s;
        s.dir  = dir;
        s.n    = (uint32_t)n1;
        s.t_is = s.t_os = s_n1;
        s.src = s.dst = tmp;
        s.others.push_back({(uint32_t)n0, s_n0, s_n0, true});
        for(size_t i = 0; i < rank; ++i)
            if(i != e)
                s.others.push_back({(uint32_t)len[i], tstride[i], tstride[i], false});
        s.others.push_back({(uint32_t)batch, tbatch, tbatch, false});
        s.flags |= FFTK_F_TWIDDLE_STORE;
        s.ltw       = ltw;
        s.ltw_shift = large_twiddle_shift(n);
        s.note      = dims_note("staged split A (fft over adjacent rows + twiddle)", n1);
        b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
    }
    // pass B: n0-point FFT over rows n1 apart in TMP, written to the user's rows k1 + n1*k0
    {
        TileSpec s;
        s.dir  = dir;
        s.n    = (uint32_t)n0;
        s.t_is = s_n0;
        s.t_os = (int64_t)n1 * out.stride[e];
        s.src  = tmp;
        s.dst  = out.io;
        s.others.push_back({(uint32_t)n1, s_n1, out.stride[e], false});
        for(size_t i = 0; i < rank; ++i)
            if(i != e)
                s.others.push_back({(uint32_t)len[i], tstride[i], out.stride[i], false});
        s.others.push_back({(uint32_t)batch, tbatch, out.stride[3], false});
        if(last_ops.has_scale)
        {
            s.flags |= FFTK_F_SCALE;
            s.scale = last_ops.scale;
        }
        s.note = dims_note("staged split B (fft over strided rows, permuted store)", n0);
        b.plan->passes.push_back(make_tile_pass(s, b.precision, b.dry));
    }
    return true;
}

// ---------------------------------------------------------------------------
// whole transforms

static std::vector<Other> other_axes(const View& in, const View& out, const size_t* len, size_t rank,
                                     size_t batch, size_t skip)
{
    std::vector<Other> o;
    for(size_t d = 0; d < rank; ++d)
        if(d != skip)
            o.push_back({(uint32_t)len[d], in.stride[d], out.stride[d]});
    o.push_back({(uint32_t)batch, in.stride[3], out.stride[3]});
    return o;
}

// Even-length real transform whose half length needs a wide kernel: the fused variant, if the
// layout allows it.  Leaves the pass list untouched and returns false otherwise.
static bool try_fused_real(Builder& b, bool forward, uint64_t half, int64_t t_is, int64_t t_os,
                           const std::vector<Other>& oth, const IoRef& src, const IoRef& dst, double scale,
                           bool has_scale)
{
    DimOps ops;
    if(forward)
        ops.store_op = FFTK_STORE_R2C_POST;
    else
        ops.load_op = FFTK_LOAD_C2R_PRE;
    ops.half_tw   = half_twiddles(half, b.precision, b.dry);
    ops.scale     = scale;
    ops.has_scale = has_scale;
    const size_t mark = b.plan->passes.size();
    try
    {
        emit_dim(b, half, t_is, t_os, oth, src, dst, forward ? -1 : +1, ops);
        return true;
    }
    catch(const PlanError&)
    {
        b.plan->passes.resize(mark);
        return false;
    }
}

static void check_sizes(const Problem& p)
{
    for(size_t d = 0; d < p.rank; ++d)
        if(p.len[d] == 0 || p.len[d] >= (1ull << 31))
            throw PlanError(rocfft_status_invalid_dimensions, "bad length");
    if(p.batch == 0 || p.batch >= (1ull << 31))
        throw PlanError(rocfft_status_failure, "bad batch");
}

static rocfft_status build_exec_plan_once(const Problem& given, ExecPlan& plan, bool dry, std::string& err)
{
    // One transform: the distances between transforms are never used, and an in-place plan may
    // name different ones for its two sides (the reference's tests do: clients/tests/
    // accuracy_test_adhoc.cpp:84-157).
    Problem p = given;
    if(p.batch == 1)
        p.idist = p.odist = 0;
    try
    {
        if(p.precision != rocfft_precision_single && p.precision != rocfft_precision_double)
            fail("half precision is not implemented");
        check_sizes(p);
        plan.passes.clear();
        plan.precision  = p.precision == rocfft_precision_double ? 1 : 0;
        plan.elem_bytes = plan.precision ? 16 : 8;
        plan.inplace    = p.placement == rocfft_placement_inplace;
        Builder b{&plan, plan.precision, dry, plan.elem_bytes};
        const int out_buf = plan.inplace ? BUF_IN : BUF_OUT;

        const bool is_real = p.type == rocfft_transform_type_real_forward
                             || p.type == rocfft_transform_type_real_inverse;
        DimOps scale_ops;
        scale_ops.scale     = p.scale;
        scale_ops.has_scale = p.has_scale;

        if(!is_real)
        {
            int  dir = p.type == rocfft_transform_type_complex_forward ? -1 : +1;
            View in  = complex_view(BUF_IN, p.in_type, p.istride, p.idist, p.ioffset, p.rank);
            View out = complex_view(out_buf, p.out_type, p.ostride, p.odist, p.ooffset, p.rank);
            if(plan.inplace)
                for(int d = 0; d < 4; ++d)
                    if(in.stride[d] != out.stride[d] && (d == 3 || (size_t)d < p.rank))
                        fail("in-place transforms need identical input and output layouts");
            size_t first = 0;
            if(emit_fused_2d(b, 0, p.len, p.rank, p.batch, in, out, dir, p.scale, p.has_scale && p.rank == 2))
                first = 2; // dimensions 0 and 1 are done
            for(size_t d = first; d < p.rank; ++d)
            {
                const View& src = d == 0 ? in : out;
                if(emit_dims_staged(b, p.len, p.rank, p.batch, d, src, out, dir,
                                    d + 2 == p.rank ? scale_ops : DimOps()))
                {
                    ++d; // dimensions d and d+1 are done
                    continue;
                }
                DimOps ops = d + 1 == p.rank ? scale_ops : DimOps();
                emit_dim(b, p.len[d], src.stride[d], out.stride[d],
                         other_axes(src, out, p.len, p.rank, p.batch, d), src.io, out.io, dir, ops);
            }
            return rocfft_status_success;
        }

        const uint64_t n0   = p.len[0];
        const uint64_t h0   = n0 / 2 + 1;
        const bool     even = n0 % 2 == 0;
        size_t         hlen[3];
        for(size_t d = 0; d < 3; ++d)
            hlen[d] = d < p.rank ? p.len[d] : 1;
        hlen[0] = h0;

        if(p.type == rocfft_transform_type_real_forward)
        {
            View hv = complex_view(out_buf, p.out_type, p.ostride, p.odist, p.ooffset, p.rank);
            bool last0 = p.rank == 1;
            // small dimensions 0 and 1: one kernel for both
            size_t next_dim = 1;
            if(even && p.rank >= 2
               && emit_fused_2d(b, 1, p.len, p.rank, p.batch,
                                realpair_view(BUF_IN, p.istride, p.idist, p.ioffset, p.rank), hv, -1, p.scale,
                                p.has_scale && p.rank == 2))
                next_dim = 2;
            else if(even && n0 >= 2)
            {
                uint64_t half = n0 / 2;
                View     rv   = realpair_view(BUF_IN, p.istride, p.idist, p.ioffset, p.rank);
                auto     oth  = other_axes(rv, hv, p.len, p.rank, p.batch, 0);
                if(half == 1)
                {
                    // two real samples a row: no transform, the post-processing step alone
                    // (bins x0 + x1 and x0 - x1) from the input to the output
                    std::vector<Other> rows;
                    for(const Other& o : oth)
                        rows.push_back({o.cnt, o.is, o.os});
                    emit_real_step(b, PASS_REAL_POST, half, rows, rv.stride[0], rv.io, hv.stride[0], hv.io, p.scale,
                                   last0 && p.has_scale);
                }
                else if(big_eligible(b, half, rv.stride[0], hv.stride[0], oth, rv.io, hv.io))
                    emit_big(b, 1, oth, rv.io, hv.io, -1, p.scale, last0 && p.has_scale);
                else if(single_kernel_length(half, b.esize)
                        && plain_dim_is_single(half, rv.stride[0] != 2, b.esize, rv.stride[0], hv.stride[0]))
                {
                    // (a half length that only the run-time-schedule kernel takes in one pass, but
                    // whose two factors have compiled kernels, goes the unfused way below)
                    DimOps ops;
                    ops.store_op = FFTK_STORE_R2C_POST;
                    ops.half_tw  = half_twiddles(half, b.precision, b.dry);
                    if(last0)
                    {
                        ops.scale     = p.scale;
                        ops.has_scale = p.has_scale;
                    }
                    emit_dim(b, half, rv.stride[0], hv.stride[0], oth, rv.io, hv.io, -1, ops);
                }
                else if(wide_kernel_length(half, b.esize)
                        && try_fused_real(b, true, half, rv.stride[0], hv.stride[0], oth, rv.io, hv.io, p.scale,
                                          last0 && p.has_scale))
                {
                    // one wide kernel with the post-processing fused
                }
                else
                {
                    // half-length complex FFT into the output rows, then the
                    // post-processing pass in place on those rows
                    emit_dim(b, half, rv.stride[0], hv.stride[0], oth, rv.io, hv.io, -1, DimOps());
                    std::vector<Other> rows;
                    for(const Other& o : oth)
                        rows.push_back({o.cnt, o.os, o.os});
                    emit_real_step(b, PASS_REAL_POST, half, rows, hv.stride[0], hv.io, hv.stride[0],
                                   hv.io, p.scale, last0 && p.has_scale);
                }
            }
            else
            {
                View   rv  = real_view(BUF_IN, p.istride, p.idist, p.ioffset, p.rank);
                auto   oth = other_axes(rv, hv, p.len, p.rank, p.batch, 0);
                DimOps ops;
                ops.load_op         = FFTK_LOAD_REAL;
                ops.src_real_scalar = true;
                ops.n_out           = (uint32_t)h0;
                if(last0)
                {
                    ops.scale     = p.scale;
                    ops.has_scale = p.has_scale;
                }
                const size_t mark = plan.passes.size();
                try
                {
                    emit_dim(b, n0, rv.stride[0], hv.stride[0], oth, rv.io, hv.io, -1, ops);
                }
                catch(const PlanError&)
                {
                    // too long for the fused real load: through a complex scratch copy
                    plan.passes.resize(mark);
                    emit_odd_real_via_complex(b, true, n0, oth, rv.stride[0], rv.io, hv.stride[0], hv.io,
                                              p.scale, last0 && p.has_scale);
                }
            }
            for(size_t d = next_dim; d < p.rank; ++d)
            {
                DimOps ops = d + 1 == p.rank ? scale_ops : DimOps();
                emit_dim(b, p.len[d], hv.stride[d], hv.stride[d],
                         other_axes(hv, hv, hlen, p.rank, p.batch, d), hv.io, hv.io, -1, ops);
            }
            return rocfft_status_success;
        }

        // real inverse: higher dimensions first, in place on the Hermitian input
        // (an out-of-place real inverse may overwrite its input: reference
        // rocfft.h:107-112, library/src/assignment_policy.cpp:601-606), then dimension 0
        View hv = complex_view(BUF_IN, p.in_type, p.istride, p.idist, p.ioffset, p.rank);
        for(size_t d = p.rank; d-- > 2;)
            emit_dim(b, p.len[d], hv.stride[d], hv.stride[d],
                     other_axes(hv, hv, hlen, p.rank, p.batch, d), hv.io, hv.io, +1, DimOps());
        // small dimensions 1 and 0: one kernel for both (it does not write to its input)
        if(even && p.rank >= 2
           && emit_fused_2d(b, 2, p.len, p.rank, p.batch, hv,
                            realpair_view(out_buf, p.ostride, p.odist, p.ooffset, p.rank), +1, p.scale,
                            p.has_scale))
            return rocfft_status_success;
        if(p.rank >= 2)
            emit_dim(b, p.len[1], hv.stride[1], hv.stride[1], other_axes(hv, hv, hlen, p.rank, p.batch, 1),
                     hv.io, hv.io, +1, DimOps());
        if(even && n0 >= 2)
        {
            uint64_t half = n0 / 2;
            View     rv   = realpair_view(out_buf, p.ostride, p.odist, p.ooffset, p.rank);
            auto     oth  = other_axes(hv, rv, p.len, p.rank, p.batch, 0);
            // in place with the standard padded rows (the real row of a bin row starts where the bin
            // row starts): the pre-processing step can run in place and leave the half-length
            // transform to whatever plan suits that length, as out of place
            bool standard_inplace = plan.inplace && !hv.io.planar && hv.stride[0] == rv.stride[0] && rv.io.im_delta == 1;
            for(int d = 1; d < 4; ++d)
                standard_inplace = standard_inplace && hv.stride[d] == rv.stride[d];
            if(half == 1)
            {
                // two real samples a row: the pre-processing step alone, from the input bins to the
                // output
                std::vector<Other> rows;
                for(const Other& o : oth)
                    rows.push_back({o.cnt, o.os, o.is});
                emit_real_step(b, PASS_REAL_PRE, half, rows, rv.stride[0], rv.io, hv.stride[0], hv.io, p.scale,
                               p.has_scale);
            }
            else if(big_eligible(b, half, hv.stride[0], rv.stride[0], oth, hv.io, rv.io))
                emit_big(b, 2, oth, hv.io, rv.io, +1, p.scale, p.has_scale);
            else if(single_kernel_length(half, b.esize)
                    && ((plan.inplace && !standard_inplace)
                        || plain_dim_is_single(half, rv.stride[0] != 2, b.esize, hv.stride[0], rv.stride[0])))
            {
                // (out of place, a half length that only the run-time-schedule kernel takes in one
                // pass but whose two factors have compiled kernels goes the unfused way below)
                DimOps ops;
                ops.load_op   = FFTK_LOAD_C2R_PRE;
                ops.half_tw   = half_twiddles(half, b.precision, b.dry);
                ops.scale     = p.scale;
                ops.has_scale = p.has_scale;
                emit_dim(b, half, hv.stride[0], rv.stride[0], oth, hv.io, rv.io, +1, ops);
            }
            else if(wide_kernel_length(half, b.esize)
                    && try_fused_real(b, false, half, hv.stride[0], rv.stride[0], oth, hv.io, rv.io, p.scale,
                                      p.has_scale))
            {
                // one wide kernel with the pre-processing fused
            }
            else
            {
                // pre-process into the output rows (viewed as half-length complex),
                // then the half-length inverse FFT in place there
                if(plan.inplace)
                {
                    bool same = !hv.io.planar && hv.stride[0] == rv.stride[0] && rv.io.im_delta == 1;
                    for(int d = 1; d < 4; ++d)
                        same = same && hv.stride[d] == rv.stride[d];
                    if(!same)
                        fail("in-place real inverse needs the standard padded layout");
                }
                std::vector<Other> rows;
                for(const Other& o : oth)
                    rows.push_back({o.cnt, o.os, o.is});
                emit_real_step(b, PASS_REAL_PRE, half, rows, rv.stride[0], rv.io, hv.stride[0], hv.io,
                               1.0, false);
                std::vector<Other> oo;
                for(const Other& o : oth)
                    oo.push_back({o.cnt, o.os, o.os});
                emit_dim(b, half, rv.stride[0], rv.stride[0], oo, rv.io, rv.io, +1, scale_ops);
            }
        }
        else
        {
            View   rv  = real_view(out_buf, p.ostride, p.odist, p.ooffset, p.rank);
            auto   oth = other_axes(hv, rv, p.len, p.rank, p.batch, 0);
            DimOps ops;
            ops.load_op         = FFTK_LOAD_HERM_EXPAND;
            ops.store_op        = FFTK_STORE_REAL;
            ops.dst_real_scalar = true;
            ops.n_in            = (uint32_t)n0;
            ops.scale           = p.scale;
            ops.has_scale       = p.has_scale;
            const size_t mark   = plan.passes.size();
            try
            {
                emit_dim(b, n0, hv.stride[0], rv.stride[0], oth, hv.io, rv.io, +1, ops);
            }
            catch(const PlanError&)
            {
                plan.passes.resize(mark);
                std::vector<Other> lines; // is = real side, os = Hermitian side
                for(const Other& o : oth)
                    lines.push_back({o.cnt, o.os, o.is});
                emit_odd_real_via_complex(b, false, n0, lines, rv.stride[0], rv.io, hv.stride[0], hv.io,
                                          p.scale, p.has_scale);
            }
        }
        return rocfft_status_success;
    }
    catch(const PlanError& e)
    {
        err = e.what();
        return e.status;
    }
    catch(const std::exception& e)
    {
        err = e.what();
        return rocfft_status_failure;
    }
}

// true when the pass has no form for buffers aligned to a scalar only
static bool needs_vector_alignment(const PassRec& r)
{
    if(r.kind == PASS_BIG || r.kind == PASS_2D)
        return true;
    return r.kind == PASS_TILE && r.kp.fast && r.kp.nthreads > 512;
}

rocfft_status build_exec_plan(const Problem& p, ExecPlan& plan, bool dry, std::string& err)
{
    rocfft_status st = build_exec_plan_once(p, plan, dry, err);
    if(st != rocfft_status_success)
        return st;
    bool any = false;
    for(const PassRec& r : plan.passes)
        any = any || needs_vector_alignment(r);
    if(any)
    {
        struct Mode
        {
            Mode()
            {
                t_generic_only = true;
            }
            ~Mode()
            {
                t_generic_only = false;
            }
        } mode;
        auto        alt = std::make_shared<ExecPlan>();
        std::string alt_err;
        // a transform the tile kernel alone cannot plan keeps the single pass list (and the
        // executor's refusal of unaligned buffers)
        if(build_exec_plan_once(p, *alt, dry, alt_err) == rocfft_status_success)
            plan.unaligned = alt;
    }
    return rocfft_status_success;
}

// ---------------------------------------------------------------------------
// executor (reference: TransformPowX, library/src/powX.cpp:525-957)

static bool aligned(const void* p, size_t a)
{
    return ((uintptr_t)p % a) == 0;
}

// a pass the run-time-schedule kernels can run with a callback on its load (first) or store (last) side
static bool pass_takes_callback(const PassRec& r, bool load_side)
{
    switch(r.kind)
    {
    case PASS_TILE:
        return r.kp.nthreads <= 512 && !r.src.planar && !r.dst.planar;
    case PASS_REAL_POST:
        return !load_side;
    case PASS_REAL_PRE:
        return load_side;
    case PASS_COPY:
        return true;
    default:
        return false;
    }
}

const ExecPlan& select_exec_plan(const ExecPlan& plan, void* const in[2], void* const out[2], const void* work,
                                 const ExecCallbacks* cb)
{
    if(!plan.unaligned)
        return plan;
    // callbacks run inside the first and last kernel: when the plan's own is a kernel without
    // callback form, the other list (run-time-schedule kernels only) takes over
    if(cb && !plan.passes.empty()
       && ((cb->load_fn && !pass_takes_callback(plan.passes.front(), true))
           || (cb->store_fn && !pass_takes_callback(plan.passes.back(), false))))
        return *plan.unaligned;
    const size_t scalar = plan.precision ? 8 : 4;
    auto         base   = [&](const IoRef& io) -> const char* {
        switch(io.buf)
        {
        case BUF_IN:
            return static_cast<const char*>(in[0]);
        case BUF_OUT:
            return static_cast<const char*>(out[0]);
        default:
            // the regions of the work buffer start at multiples of the element size
            return static_cast<const char*>(work);
        }
    };
    for(const PassRec& rec : plan.passes)
    {
        if(!needs_vector_alignment(rec))
            continue;
        const size_t need = rec.kind == PASS_BIG ? 8 : plan.elem_bytes;
        const char*  s0   = base(rec.src);
        const char*  d0   = base(rec.dst);
        if((s0 && !aligned(s0 + rec.src.off0 * (int64_t)scalar, need))
           || (d0 && !aligned(d0 + rec.dst.off0 * (int64_t)scalar, need)))
            return *plan.unaligned;
    }
    return plan;
}

bool callbacks_fusable(const ExecPlan& plan, void* const in[2], void* const out[2], const void* work,
                       const ExecCallbacks& cb)
{
    const ExecPlan& chosen = select_exec_plan(plan, in, out, work, &cb);
    if(chosen.passes.empty())
        return false;
    if(cb.load_fn && !pass_takes_callback(chosen.passes.front(), true))
        return false;
    if(cb.store_fn && !pass_takes_callback(chosen.passes.back(), false))
        return false;
    return true;
}

// the passes whose user side may be an array of half pairs: what variant 6 of the compiled
// kernels covers (fast_kernels.hip)
static bool pass_takes_half(const PassRec& r)
{
    if(r.kind != PASS_TILE || !r.kp.fast || !r.lean_ok)
        return false;
    const fftk_params& k = r.kp;
    return (k.load_op == FFTK_LOAD_COMPLEX || k.load_op == FFTK_LOAD_C2R_PRE)
           && (k.store_op == FFTK_STORE_COMPLEX || k.store_op == FFTK_STORE_R2C_POST)
           && (k.flags & ~(uint32_t)(FFTK_F_SCALE | FFTK_F_TWIDDLE_STORE)) == 0 && !k.in_planar && !k.out_planar
           && !k.w_inner && k.n_in == k.n && k.n_out == k.n && fftrt_fast_takes_half(k.n) != 0;
}

bool half_fusable(const ExecPlan& plan, bool input, const void* user)
{
    if(plan.precision != 0 || plan.passes.empty() || !user)
        return false;
    const PassRec& r  = input ? plan.passes.front() : plan.passes.back();
    const IoRef&   io = input ? r.src : r.dst;
    const int      want = input || plan.inplace ? BUF_IN : BUF_OUT;
    if(!pass_takes_half(r) || io.buf != want || io.planar || io.im_delta != 1)
        return false;
    if(input)
    {
        // every later pass that reads the input array must find it rewritten (in single
        // precision, in the scratch copy) by an earlier one
        bool rewritten = false;
        for(size_t i = 0; i < plan.passes.size(); ++i)
        {
            if(i > 0 && plan.passes[i].src.buf == BUF_IN && !rewritten)
                return false;
            if(plan.passes[i].dst.buf == BUF_IN)
                rewritten = true;
        }
    }
    // a pair of half values is one 4-byte access
    return ((uintptr_t)(static_cast<const char*>(user) + io.off0 * 2) % 4) == 0;
}

void half_scratch_needs(const ExecPlan& plan, bool fuse_in, bool fuse_out, bool& need_in, bool& need_out)
{
    need_in = need_out = false;
    const size_t n = plan.passes.size();
    for(size_t i = 0; i < n; ++i)
    {
        const PassRec& r     = plan.passes[i];
        const bool     first = i == 0, last = i + 1 == n;
        if(r.src.buf == BUF_IN && !(first && fuse_in))
            need_in = true;
        if(r.src.buf == BUF_OUT)
            need_out = true;
        // (in place the output array is the input array; out of place a real inverse transform
        // may still work on its input array)
        if(r.dst.buf == BUF_OUT && !(last && fuse_out))
            need_out = true;
        if(r.dst.buf == BUF_IN && !(plan.inplace && last && fuse_out))
            need_in = true;
    }
    if(plan.inplace)
        need_in = need_out = need_in || need_out;
}

// Single-precision passes that move far more data than the last-level cache holds (256 MB) read
// and write interleaved arrays with the nontemporal hint: nothing they touch is used again
// before it would be evicted anyway.  Measured on MI355X: 4096 x 4096 x 8 transform 1.31 -> 1.23 ms,
// 65536 rows of 4096 points 0.81 -> 0.79 ms.  Only where every contiguous run of a tile on that
// side starts and ends on a 128-byte line: on tiles that share lines with their neighbours the
// hint keeps the halves from merging in the cache (512 x 512 x 257 double-precision columns,
// 257 bins a row: 0.43 -> 0.84 ms), and double-precision passes measured 3-8 % slower with it.
// And only where every access of a wave covers whole lines: along a transform the lanes of one
// transform read neighbouring elements, so with fewer than 128 bytes of lanes a transform a line
// is fetched piecewise by several instructions, and with the hint once for each of them (rows
// of 32 points, 2 threads a transform, 1 GB: 0.48 -> 2.65 ms).
static const double NT_MIN_MBYTES = 768.0;
static bool pass_streams_side(const fftk_params& k, bool in)
{
    const int64_t line = 32; // scalars of 4 bytes per 128-byte line
    if((in ? k.in_planar : k.out_planar) || k.w_inner)
        return false;
    const int64_t  t = in ? k.t_is : k.t_os, w = in ? k.w_is : k.w_os;
    const bool     fast_tile = in ? k.in_fast_tile != 0 : k.out_fast_tile != 0;
    const int64_t* o = in ? k.o_is : k.o_os;
    for(int i = 0; i < 3; ++i)
        if(k.oc[i] > 1 && o[i] % line)
            return false;
    if(fast_tile) // runs of W elements along the tile axis
        return w == 2 && (k.W * 2) % line == 0 && t % line == 0 && k.tile_cnt % k.W == 0;
    // runs of n elements along the transform, T lanes of a transform side by side (or the tile
    // copied through LDS by consecutive lanes)
    if(!k.stage_io && ((int64_t)k.T * 2) % line)
        return false;
    return t == 2 && ((int64_t)k.n * 2) % line == 0 && (k.tile_cnt == 1 || w % line == 0);
}

rocfft_status run_exec_plan(const ExecPlan& plan, void* const in[2], void* const out[2], void* work,
                            void* stream, float* pass_ms, const ExecCallbacks* cb, const ExecHalf* half)
{
    {
        const ExecPlan& chosen = select_exec_plan(plan, in, out, work, cb);
        if(&chosen != &plan)
        {
            if(half && (half->fuse_in || half->fuse_out))
                return rocfft_status_failure; // (decided for the primary list: the caller checks)
            // (per-pass timings describe the primary pass list: not reported for the other one)
            if(pass_ms)
                for(size_t i = 0; i < plan.passes.size(); ++i)
                    pass_ms[i] = -1.0f;
            return run_exec_plan(chosen, in, out, work, stream, nullptr, cb);
        }
    }
    // the callback descriptor of a pass: the load callback belongs to the first pass, the
    // store callback to the last one; every other access is plain
    const size_t npass = plan.passes.size();
    auto         cb_of = [&](size_t index, const IoRef& src, const IoRef& dst, fftk_cb& d) {
        memset(&d, 0, sizeof(d));
        if(!cb)
            return false;
        bool any = false;
        if(cb->load_fn && index == 0)
        {
            d.load_fn    = cb->load_fn;
            d.load_data  = cb->load_data;
            d.in_base    = in[0];
            d.in_off     = src.off0;
            d.in_complex = cb->in_complex ? 1 : 0;
            any          = true;
        }
        if(cb->store_fn && index + 1 == npass)
        {
            d.store_fn    = cb->store_fn;
            d.store_data  = cb->store_data;
            d.out_base    = out[0];
            d.out_off     = dst.off0;
            d.out_complex = cb->out_complex ? 1 : 0;
            any           = true;
        }
        return any;
    };
    const size_t scalar = plan.precision ? 8 : 4;
    char*        tmp    = static_cast<char*>(work);
    char*        blu    = tmp ? tmp + plan.tmp_elems * plan.elem_bytes : nullptr;
    char*        cpx    = tmp ? blu + plan.blu_elems * plan.elem_bytes : nullptr;
    auto resolve = [&](const IoRef& io, char*& p0, char*& p1) -> bool {
        char* base0 = nullptr;
        char* base1 = nullptr;
        switch(io.buf)
        {
        case BUF_IN:
            base0 = static_cast<char*>(in[0]);
            base1 = static_cast<char*>(in[1]);
            break;
        case BUF_OUT:
            base0 = static_cast<char*>(out[0]);
            base1 = static_cast<char*>(out[1]);
            break;
        case BUF_TMP:
            base0 = tmp;
            break;
        case BUF_CPX:
            base0 = cpx;
            break;
        default:
            base0 = blu;
            break;
        }
        if(!base0)
            return false;
        p0 = base0 + io.off0 * (int64_t)scalar;
        if(io.planar)
        {
            if(!base1)
                return false;
            p1 = base1 + io.off1 * (int64_t)scalar;
        }
        else
            p1 = p0 + io.im_delta * (int64_t)scalar;
        return true;
    };
    // optional per-pass timing (the reference's profile layer does the same with
    // hipEvents around every kernel, library/src/powX.cpp:817-883)
    struct Events
    {
        std::vector<void*> v;
        ~Events()
        {
            for(void* e : v)
                if(e)
                    fftrt_event_destroy(e);
        }
    } ev;
    std::vector<void*>& events = ev.v;
    if(pass_ms)
    {
        events.resize(plan.passes.size() + 1, nullptr);
        for(void*& e : events)
            if(fftrt_event_create(&e) != 0)
                return rocfft_status_failure;
        fftrt_event_record(events[0], stream);
    }
    size_t pass_index = 0;
    for(const PassRec& rec : plan.passes)
    {
        char *s0, *s1, *d0, *d1;
        if(!resolve(rec.src, s0, s1) || !resolve(rec.dst, d0, d1))
            return rocfft_status_failure;
        int rc;
        if(rec.kind == PASS_BIG || rec.kind == PASS_2D)
        {
            fftk_cb none;
            if(cb_of(pass_index, rec.src, rec.dst, none))
                return rocfft_status_failure; // these kernels have no callback form
        }
        if(rec.kind == PASS_BIG)
        {
            fftk_big_params q = rec.bp;
            q.in              = s0;
            q.out             = d0;
            if(!aligned(s0, 8) || !aligned(d0, 8))
                return rocfft_status_failure;
            rc = fftrt_launch_big32k(&q, stream);
        }
        else if(rec.kind == PASS_2D)
        {
            fftk_params k = rec.kp;
            k.in0         = s0;
            k.in1         = s1;
            k.out0        = d0;
            k.out1        = d1;
            if(!aligned(s0, plan.elem_bytes) || !aligned(d0, plan.elem_bytes))
                return rocfft_status_failure;
            if(k.store_op == FFTK_STORE_R2C_POST || k.load_op == FFTK_LOAD_C2R_PRE)
                rc = fftrt_launch_fast2d_real(&k, plan.precision, k.load_op == FFTK_LOAD_C2R_PRE ? 1 : 0, rec.grid,
                                              rec.lds, stream);
            else
                rc = fftrt_launch_fast2d(&k, plan.precision, rec.grid, rec.lds, stream);
        }
        else if(rec.kind == PASS_COPY)
        {
            fftk_copy_params c = rec.cp;
            c.s0               = s0;
            c.s1               = s1;
            c.d0               = d0;
            c.d1               = d1;
            cb_of(pass_index, rec.src, rec.dst, c.cb);
            rc                 = fftrt_launch_copy(&c, plan.precision, stream);
        }
        else if(rec.kind == PASS_TILE)
        {
            fftk_params k = rec.kp;
            k.in0         = s0;
            k.in1         = s1;
            k.out0        = d0;
            k.out1        = d1;
            bool vec = rec.vec_ok && aligned(s0, plan.elem_bytes) && aligned(d0, plan.elem_bytes);
            k.lean   = 0;
            if(rec.lean_ok)
            {
                // interleaved complex sides need the alignment of a pair, planar and real sides that
                // of a scalar
                const size_t in_al  = (k.in_planar || k.load_op == FFTK_LOAD_REAL) ? plan.elem_bytes / 2 : plan.elem_bytes;
                const size_t out_al = (k.out_planar || k.store_op == FFTK_STORE_REAL) ? plan.elem_bytes / 2 : plan.elem_bytes;
                k.lean = (aligned(s0, in_al) && aligned(d0, out_al) && (!k.in_planar || aligned(s1, in_al))
                          && (!k.out_planar || aligned(d1, out_al)))
                             ? 1
                             : 0;
            }
            const bool with_cb = cb_of(pass_index, rec.src, rec.dst, k.cb);
            if(with_cb)
            {
                // the run-time-schedule kernel runs the same schedule and calls the callbacks
                if(!pass_takes_callback(rec, pass_index == 0 && cb->load_fn))
                    return rocfft_status_failure;
                k.fast = 0;
                k.lean = 0;
            }
            if(half && ((half->fuse_in && pass_index == 0) || (half->fuse_out && pass_index + 1 == npass)))
            {
                // the user's half array in place of the scratch copy on that side
                if(half->fuse_in && pass_index == 0)
                {
                    k.in0     = static_cast<char*>(half->in) + rec.src.off0 * 2;
                    k.in1     = static_cast<const char*>(k.in0) + 2;
                    k.in_half = 1;
                }
                if(half->fuse_out && pass_index + 1 == npass)
                {
                    k.out0     = static_cast<char*>(half->out) + rec.dst.off0 * 2;
                    k.out1     = static_cast<char*>(k.out0) + 2;
                    k.out_half = 1;
                }
                // the other side is a scratch array of the plan (aligned)
                if(!rec.lean_ok || with_cb || (!k.in_half && !aligned(k.in0, plan.elem_bytes))
                   || (!k.out_half && !aligned(k.out0, plan.elem_bytes)))
                    return rocfft_status_failure;
                k.lean = 1;
            }
            // Nontemporal accesses (see pass_streams_side): ROCFFT_AMD_NO_NT=1 switches them off,
            // ROCFFT_AMD_NT_MB sets the least data volume of a pass in megabytes (comparisons)
            {
                static const bool   nt_on  = !getenv("ROCFFT_AMD_NO_NT");
                static const double nt_min = (getenv("ROCFFT_AMD_NT_MB") ? atof(getenv("ROCFFT_AMD_NT_MB")) : NT_MIN_MBYTES) * 1e6;
                if(nt_on && k.lean && plan.precision == 0 && rec.bytes_rw >= nt_min && !with_cb)
                {
                    k.in_nt  = pass_streams_side(k, true) && !k.in_half && aligned(k.in0, 128) ? 1 : 0;
                    k.out_nt = pass_streams_side(k, false) && !k.out_half && aligned(k.out0, 128) ? 1 : 0;
                }
            }
            rc = fftrt_launch_tile(&k, plan.precision, vec ? 1 : 0, rec.grid, rec.lds, stream);
        }
        else
        {
            fftk_real_params r = rec.rp;
            if(cb_of(pass_index, rec.src, rec.dst, r.cb)
               && !pass_takes_callback(rec, pass_index == 0 && cb->load_fn))
                return rocfft_status_failure;
            if(rec.kind == PASS_REAL_POST)
            {
                r.z0  = s0;
                r.z1  = s1;
                r.ho0 = d0;
                r.ho1 = d1;
                rc    = fftrt_launch_real_post(&r, plan.precision, stream);
            }
            else
            {
                r.h0  = s0;
                r.h1  = s1;
                r.zo0 = d0;
                r.zo1 = d1;
                rc    = fftrt_launch_real_pre(&r, plan.precision, stream);
            }
        }
        if(rc != 0)
            return rocfft_status_failure;
        ++pass_index;
        if(pass_ms)
            fftrt_event_record(events[pass_index], stream);
    }
    if(pass_ms)
    {
        for(size_t i = 0; i < plan.passes.size(); ++i)
            if(fftrt_event_elapsed_ms(events[i], events[i + 1], &pass_ms[i]) != 0)
                pass_ms[i] = -1.0f;
    }
    return rocfft_status_success;
}

static const char* buf_name(int b)
{
    switch(b)
    {
    case BUF_IN:
        return "in";
    case BUF_OUT:
        return "out";
    case BUF_TMP:
        return "tmp";
    case BUF_CPX:
        return "cpx";
    default:
        return "blu";
    }
}

std::string ExecPlan::describe() const
{
    std::ostringstream o;
    o << "plan: " << passes.size() << " passes, precision " << (precision ? "double" : "single")
      << ", work buffer " << work_bytes() << " bytes\n";
    int i = 0;
    for(const PassRec& r : passes)
    {
        o << "  pass " << i++ << ": " << r.note << " [" << buf_name(r.src.buf) << " -> "
          << buf_name(r.dst.buf) << "]";
        if(r.kind == PASS_TILE)
        {
            const fftk_params& k = r.kp;
            o << " radix";
            for(uint32_t p = 0; p < k.nf; ++p)
                o << (p ? "x" : " ") << k.radix[p];
            o << " tile " << k.W << "x" << k.n << " threads " << k.nthreads << " grid " << r.grid
              << " lds " << r.lds << " in_fast_" << (k.in_fast_tile ? "tile" : "fft") << " out_fast_"
              << (k.out_fast_tile ? "tile" : "fft") << " flags 0x" << std::hex << k.flags << std::dec
              << " load " << k.load_op << " store " << k.store_op << (r.vec_ok ? " vec" : " scalar");
            if(r.lean_ok)
                o << " lean" << (k.in_planar ? " planar_in" : "") << (k.out_planar ? " planar_out" : "");
            if(k.xcd_remap)
                o << " xcd_ranges";
            if(k.oc0_first)
                o << " batch_first";
            if(k.w_inner)
                o << " folded(" << k.w_inner << ")";
            if(k.fast)
                o << " fast" << (k.direct_in ? " direct_in" : " staged_in")
                  << (k.direct_out ? " direct_out" : " staged_out") << (k.stage_io ? " tile_copy" : "");
        }
        else if(r.kind == PASS_BIG)
            o << " threads 1024 grid " << r.grid << " lds 135296";
        else if(r.kind == PASS_COPY)
            o << " rows " << r.cp.rows0 << "x" << r.cp.rows1 << "x" << r.cp.rows2;
        else if(r.kind == PASS_2D)
            o << " tile " << r.kp.W << "x" << r.kp.n << "x" << r.kp.n2 << " threads " << r.kp.nthreads << " grid "
              << r.grid << " lds " << r.lds;
        else
            o << " half " << r.rp.half << " rows " << r.rp.rows0 << "x" << r.rp.rows1 << "x"
              << r.rp.rows2;
        o << "\n";
    }
    if(unaligned)
        o << "  for buffers without vector alignment: " << unaligned->passes.size() << " passes, work buffer "
          << unaligned->own_work_bytes() << " bytes\n";
    return o.str();
}

} // namespace fftamd
