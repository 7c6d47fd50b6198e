// big_kernels.hip -- one-workgroup 32768-point single-precision FFT.
//
// A 32768-point complex transform (256 KB in fp32) does not fit the 160 KB LDS of
// a compute unit, but it fits the register file: 1024 threads hold 32 complex
// values each.  The three radix-32 passes exchange data through LDS one scalar
// plane at a time (real parts, then imaginary parts: 128 KB + padding), so the
// transform makes exactly one trip through HBM.  Even-length real transforms of
// 65536 points use it with the pre-/post-processing fused in:
//   real forward : real pairs in -> FFT -> Hermitian post-processing -> 32769 bins
//   real inverse : 32769 bins -> pre-processing -> inverse FFT -> real pairs out
// The reference needs three kernels and three trips through HBM for each of
// these (SBCC-128, SBRC-256, r2c_even_post; library/src/node_factory.cpp:42-51,
// library/src/tree_node_real.cpp:263-279).  The pre/post formulas are those of
// library/src/device/kernels/real2complex_device.h:25-103, :212-254.
#include "butterfly.h"
#include "gpu_rt.h"
#include "kparams.h"
#include "lds_limit.h"
#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>

namespace
{

constexpr int BIG_L       = 32768;
constexpr int BIG_THREADS = 1024;
constexpr int BIG_EPT     = 32;

template <typename T>
struct Butterfly32
{
    typedef typename cplx_of<T>::type C;
    // n = n1 + 4 n2, k = 8 k1 + k2:
    //   y[n1][k2] = sum_n2 x[n1 + 4 n2] W_8^{n2 k2};  X[8 k1 + k2] = sum_n1 W_4^{n1 k1} W_32^{n1 k2} y[n1][k2]
    // first stage: four radix-8 groups (group n1 works on slots n1 + 4 n2) and the W_32 twiddles
    static __device__ __forceinline__ void stage_a(C* r)
    {
        // cos/sin(2 pi m/32), m = 0..8
        const T cs[9] = {(T)1.0,
                         (T)0.980785280403230449126182236134239037,
                         (T)0.923879532511286756128183189396788287,
                         (T)0.831469612302545237078788377617905757,
                         (T)0.707106781186547524400844362104849039,
                         (T)0.555570233019602224742830813948532874,
                         (T)0.382683432365089771728459984030398866,
                         (T)0.195090322016128267848284868477022240,
                         (T)0.0};
#pragma unroll
        for(int n1 = 0; n1 < 4; ++n1)
        {
            C y[8];
#pragma unroll
            for(int n2 = 0; n2 < 8; ++n2)
                y[n2] = r[n1 + 4 * n2];
            Butterfly<T, 8>::run(y);
#pragma unroll
            for(int k2 = 0; k2 < 8; ++k2)
            {
                // W_32^{n1 k2}, exponent at most 21
                const int m = n1 * k2;
                C         v = y[k2];
                if(m != 0)
                {
                    // cos(2 pi m/32), -sin(2 pi m/32) from the first-quadrant table
                    T co, si;
                    if(m <= 8)
                    {
                        co = cs[m];
                        si = cs[8 - m];
                    }
                    else if(m <= 16)
                    {
                        co = -cs[16 - m];
                        si = cs[m - 8];
                    }
                    else
                    {
                        co = -cs[m - 16];
                        si = -cs[24 - m];
                    }
                    C t;
                    t.x = v.x * co + v.y * si;
                    t.y = v.y * co - v.x * si;
                    v   = t;
                }
                r[n1 + 4 * k2] = v; // slot (n1, k2)
            }
        }
    }
    // second stage, group k2: a radix-4 butterfly on slots 4 k2 .. 4 k2 + 3, which then hold
    // X[8 k1 + k2] in slot k1 + 4 k2 (see big_slot_index)
    static __device__ __forceinline__ void stage_b(C* r, int k2)
    {
        C z[4] = {r[0 + 4 * k2], r[1 + 4 * k2], r[2 + 4 * k2], r[3 + 4 * k2]};
        Butterfly<T, 4>::run(z);
        r[0 + 4 * k2] = z[0];
        r[1 + 4 * k2] = z[1];
        r[2 + 4 * k2] = z[2];
        r[3 + 4 * k2] = z[3];
    }
    static __device__ __forceinline__ void run(C* r)
    {
        stage_a(r);
#pragma unroll
        for(int k2 = 0; k2 < 8; ++k2)
            stage_b(r, k2);
    }
};

// Butterfly32 leaves output X[8 k1 + k2] in slot k1 + 4 k2
__device__ __forceinline__ constexpr int big_slot_index(int s)
{
    return 8 * (s & 3) + (s >> 2);
}

// Padded LDS index of scalar i is i + (i >> 5) (one pad word per 32).  With t < 1024 and
// k < 32 the three access patterns reduce to a per-thread base plus a compile-time offset:
//   i = 32 t + k              -> 33 t + k
//   i = t + 1024 k            -> t + (t >> 5) + 1056 k
//   i = (t/32) 1024 + t%32 + 32 k -> (t >> 5) 1056 + (t & 31) + 33 k

// r[k] *= w^k for k = 1..31 with w^1..w^7 and w^8, w^16, w^24 read from the stacked
// table of the pass (entry (k-1)*c + bl) and the rest formed as w^(8a) * w^b
template <typename C>
struct BigTwiddle
{
    C lo[8]; // w^1 .. w^7 in lo[1..7]
    C hi[4]; // w^8, w^16, w^24 in hi[1..3]
    __device__ __forceinline__ void load(const C* tw, uint32_t c, uint32_t bl)
    {
#pragma unroll
        for(int k = 1; k < 8; ++k)
            lo[k] = tw[(k - 1) * c + bl];
#pragma unroll
        for(int a = 1; a < 4; ++a)
            hi[a] = tw[(8 * a - 1) * c + bl];
    }
    __device__ __forceinline__ void apply(C* r) const
    {
#pragma unroll
        for(int k = 1; k < 8; ++k)
            r[k] = c_mul(r[k], lo[k]);
#pragma unroll
        for(int a = 1; a < 4; ++a)
        {
            r[8 * a] = c_mul(r[8 * a], hi[a]);
#pragma unroll
            for(int b = 1; b < 8; ++b)
                r[8 * a + b] = c_mul(r[8 * a + b], c_mul(hi[a], lo[b]));
        }
    }
};

template <typename C>
__device__ __forceinline__ void big_twiddle(C* r, const C* tw, uint32_t c, uint32_t bl)
{
    BigTwiddle<C> w;
    w.load(tw, c, bl);
    w.apply(r);
}

// e^{-2 pi i k/64}, k = 0..15.  The pre-/post-processing twiddle of bin j = t + 1024 k is
// e^{-2 pi i t/65536} e^{-2 pi i k/64}; the second factor belongs to the register slot and is
// read through the scalar cache into scalar registers (constant address space: no vector
// memory instruction, nothing for the vector memory counter to wait on).
__constant__ float2 BIG_W64[16] = {
    {1.000000000000000000000000e+00f, -0.000000000000000000000000e+00f},
    {9.951847266721969287317506e-01f, -9.801714032956060362877793e-02f},
    {9.807852804032304305792422e-01f, -1.950903220161282480837883e-01f},
    {9.569403357322088243819280e-01f, -2.902846772544623310530199e-01f},
    {9.238795325112867384831361e-01f, -3.826834323650897817792327e-01f},
    {8.819212643483550495560053e-01f, -4.713967368259976420397095e-01f},
    {8.314696123025452356714027e-01f, -5.555702330196021776487214e-01f},
    {7.730104533627369933768136e-01f, -6.343932841636454877942697e-01f},
    {7.071067811865475727373109e-01f, -7.071067811865474617150085e-01f},
    {6.343932841636454877942697e-01f, -7.730104533627369933768136e-01f},
    {5.555702330196022886710239e-01f, -8.314696123025452356714027e-01f},
    {4.713967368259978085731632e-01f, -8.819212643483549385337028e-01f},
    {3.826834323650898372903839e-01f, -9.238795325112867384831361e-01f},
    {2.902846772544623310530199e-01f, -9.569403357322089354042305e-01f},
    {1.950903220161283313505152e-01f, -9.807852804032304305792422e-01f},
    {9.801714032956077016223162e-02f, -9.951847266721968177094482e-01f}};

__device__ __forceinline__ float2 big_w64(int k)
{
    return BIG_W64[k];
}

typedef fftk_big_params big_params;

template <int MODE>
__global__ __launch_bounds__(BIG_THREADS) void big32k_kernel(const big_params p)
{
    extern __shared__ float lds[];
    float2*                 lds2 = reinterpret_cast<float2*>(lds); // 16384 complex values
    const uint32_t          t    = threadIdx.x;
    uint32_t                b    = blockIdx.x;
    const uint32_t          l0   = b % p.lines[0];
    b /= p.lines[0];
    const uint32_t l1 = b % p.lines[1];
    const uint32_t l2 = b / p.lines[1];
    const float*   in = static_cast<const float*>(p.in) + l0 * p.in_line[0] + l1 * p.in_line[1]
                      + l2 * p.in_line[2];
    float* out = static_cast<float*>(p.out) + l0 * p.out_line[0] + l1 * p.out_line[1]
                 + l2 * p.out_line[2];
    const float2* tw  = static_cast<const float2*>(p.tw);
    const bool    inv = MODE == 2 || (MODE == 0 && p.dir > 0);
    constexpr int HALF = BIG_L / 2;

    float2 r[BIG_EPT];
    // ---- load: slot k holds element j = t + 1024 k
    if(MODE != 2)
    {
#pragma unroll
        for(int k = 0; k < BIG_EPT; ++k)
        {
            // wave-uniform base per k plus the lane offset t: no per-element address registers
            float2 v = (reinterpret_cast<const float2*>(in) + 1024 * k)[t];
            r[k]     = inv ? c_swap(v) : v;
        }
    }
    else
    {
        // Hermitian bins -> half-length complex input.  The owner of j < L/2 loads X_j and
        // X_{L-j} (every bin is loaded once), forms z_j and z_{L-j}, keeps the first and hands
        // the second to its owner through LDS.  Only the real parts of bins 0 and L are used.
        const float2  a  = static_cast<const float2*>(p.half_a)[t];
        const float2* hx = reinterpret_cast<const float2*>(in);
        const uint32_t tr = 1023u - t;
#pragma unroll
        for(int k = 0; k < BIG_EPT / 2; ++k)
        {
            const uint32_t j  = t + 1024 * k;
            float2         xa = (hx + 1024 * k)[t];
            float2         xb = (hx + (BIG_L - 1024 * k - 1023))[tr];
            float2         zj, zq;
            if(k == 0 && t == 0)
            {
                zj.x = xa.x + xb.x;
                zj.y = xa.x - xb.x;
                r[k] = c_swap(zj);
            }
            else
            {
                float2 tj = c_mul(a, big_w64(k));
                float2 u, v;
                u.x  = xa.x + xb.x;
                u.y  = xa.y + xb.y;
                v.x  = xa.x - xb.x;
                v.y  = xa.y - xb.y;
                zj.x = u.x + v.x * tj.y - u.y * tj.x;
                zj.y = v.y + u.y * tj.y + v.x * tj.x;
                zq.x = u.x - v.x * tj.y + u.y * tj.x;
                zq.y = -v.y + u.y * tj.y + v.x * tj.x;
                r[k] = c_swap(zj);
                lds2[HALF - j] = c_swap(zq);
            }
        }
        if(t == 0)
        {
            float2 xm = hx[HALF];
            float2 zm;
            zm.x    = 2.0f * xm.x;
            zm.y    = -2.0f * xm.y;
            lds2[0] = c_swap(zm);
        }
        __syncthreads();
#pragma unroll
        for(int k = BIG_EPT / 2; k < BIG_EPT; ++k)
            r[k] = lds2[t + 1024 * (k - BIG_EPT / 2)];
        __syncthreads();
    }

    const uint32_t w1base = 33 * t;
    const uint32_t rbase  = t + (t >> 5);
    const uint32_t w2base = (t >> 5) * 1056 + (t & 31);
    // ---- pass 0 (outputs in slot order: slot s holds output big_slot_index(s))
    Butterfly32<float>::run(r);
    // exchange 1: write 32 t + k_out, read t + 1024 k
#pragma unroll
    for(int s = 0; s < BIG_EPT; ++s)
        lds[w1base + big_slot_index(s)] = r[s].x;
    __syncthreads();
#pragma unroll
    for(int k = 0; k < BIG_EPT; ++k)
        r[k].x = lds[rbase + 1056 * k];
    __syncthreads();
#pragma unroll
    for(int s = 0; s < BIG_EPT; ++s)
        lds[w1base + big_slot_index(s)] = r[s].y;
    __syncthreads();
#pragma unroll
    for(int k = 0; k < BIG_EPT; ++k)
        r[k].y = lds[rbase + 1056 * k];
    // ---- pass 1 (cumulative height 32)
    {
        const uint32_t bl = t & 31u;
#pragma unroll
        for(int k = 1; k < BIG_EPT; ++k)
            r[k] = c_mul(r[k], tw[(k - 1) * 32 + bl]);
    }
    Butterfly32<float>::run(r);
    __syncthreads();
    // exchange 2: write (t/32)*1024 + (t%32) + 32 k_out, read t + 1024 k
#pragma unroll
    for(int s = 0; s < BIG_EPT; ++s)
        lds[w2base + 33 * big_slot_index(s)] = r[s].x;
    __syncthreads();
#pragma unroll
    for(int k = 0; k < BIG_EPT; ++k)
        r[k].x = lds[rbase + 1056 * k];
    __syncthreads();
#pragma unroll
    for(int s = 0; s < BIG_EPT; ++s)
        lds[w2base + 33 * big_slot_index(s)] = r[s].y;
    __syncthreads();
#pragma unroll
    for(int k = 0; k < BIG_EPT; ++k)
        r[k].y = lds[rbase + 1056 * k];
    // ---- pass 2 (cumulative height 1024); stacked offset of pass 2 is 31*32
    big_twiddle(r, tw + 31 * 32, 1024u, t);
    Butterfly32<float>::run(r);
    // slot s holds Z[t + 1024 big_slot_index(s)] (re/im exchanged when inverse)

    if(MODE != 1)
    {
#pragma unroll
        for(int s = 0; s < BIG_EPT; ++s)
        {
            float2 v = inv ? c_swap(r[s]) : r[s];
            if(p.use_scale)
            {
                v.x *= (float)p.scale;
                v.y *= (float)p.scale;
            }
            (reinterpret_cast<float2*>(out) + 1024 * big_slot_index(s))[t] = v;
        }
        return;
    }

    // ---- real forward: the owner of j < L/2 fetches Z_{L-j} from its owner through LDS and
    // writes both X_j and X_{L-j}
    __syncthreads();
#pragma unroll
    for(int s = 0; s < BIG_EPT; ++s)
        if(big_slot_index(s) >= BIG_EPT / 2)
            lds2[t + 1024 * (big_slot_index(s) - BIG_EPT / 2)] = r[s];
    __syncthreads();
    const float2  a  = static_cast<const float2*>(p.half_a)[t];
    float2*       ho = reinterpret_cast<float2*>(out);
    const float   sc = p.use_scale ? (float)p.scale : 1.0f;
    const uint32_t tr = 1023u - t;
#pragma unroll
    for(int s = 0; s < BIG_EPT; ++s)
    {
        const int k = big_slot_index(s);
        if(k >= BIG_EPT / 2)
        {
            if(k == BIG_EPT / 2 && t == 0)
            {
                // bin L/2 pairs with itself
                float2 o;
                o.x      = r[s].x * sc;
                o.y      = -r[s].y * sc;
                ho[HALF] = o;
            }
            continue;
        }
        const uint32_t j  = t + 1024 * k;
        float2         zp = r[s];
        float2         o0, o1;
        if(k == 0 && t == 0)
        {
            o0.x = zp.x + zp.y;
            o0.y = 0.0f;
            o1.x = zp.x - zp.y;
            o1.y = 0.0f;
        }
        else
        {
            float2 zq = lds2[HALF - j];
            float2 tj = c_mul(a, big_w64(k));
            float2 u, v;
            u.x  = 0.5f * (zp.x + zq.x);
            u.y  = 0.5f * (zp.y + zq.y);
            v.x  = 0.5f * (zp.x - zq.x);
            v.y  = 0.5f * (zp.y - zq.y);
            o0.x = u.x + v.x * tj.y + u.y * tj.x;
            o0.y = v.y + u.y * tj.y - v.x * tj.x;
            o1.x = u.x - v.x * tj.y - u.y * tj.x;
            o1.y = -v.y + u.y * tj.y - v.x * tj.x;
        }
        o0.x *= sc;
        o0.y *= sc;
        o1.x *= sc;
        o1.y *= sc;
        (ho + 1024 * k)[t]                   = o0;
        (ho + (BIG_L - 1024 * k - 1023))[tr] = o1;
    }
}

// ---------------------------------------------------------------------------
// Streaming variant: one workgroup per compute unit walks through the transforms and,
// while it runs the last pass and the stores of one transform, has part of the next
// transform copied from global memory straight into LDS (asynchronous global -> LDS
// loads, no registers involved).  A compute unit can hold one transform only, so without
// this its memory pipes idle during the arithmetic and its arithmetic idles during the loads.
//
// A chunk = 1024 consecutive complex values = one register slot of every thread.
//   complex, real forward: chunks 0,1,4,5,8,9,... go through LDS: the operands of the first
//     radix-8 groups of pass 0, which start while the other chunks are still in flight.
//   real inverse: the first 16384 bins go through LDS, their partners X_{L-j} come straight
//     from global memory.
// LDS (floats): the exchanges between passes use [0, 33792); the prefetch area starts at
// PF_BASE and is filled after the last exchange of the previous transform; the real forward
// transform keeps [0, 16384) for the pairwise hand-over of its post-processing, which runs
// in two rounds of 8 values per thread while the prefetch is already under way.

typedef const __attribute__((address_space(1))) void* big_gptr;
typedef __attribute__((address_space(3))) void*       big_lptr;

__device__ __forceinline__ constexpr int big_pf_chunk(int s)
{
    return 4 * (s >> 1) + (s & 1);
}

__device__ __forceinline__ constexpr bool big_chunk_prefetched(int k, int pf)
{
    for(int s = 0; s < pf; ++s)
        if(big_pf_chunk(s) == k)
            return true;
    return false;
}

// workgroup barrier that orders LDS traffic only (global loads and stores stay in flight)
__device__ __forceinline__ void big_lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Copies PF chunks of the row to LDS, 16 bytes per lane (src must be 16-byte aligned): copy
// number id = 0 .. 8 PF - 1 moves 1 KB, the copies are dealt out evenly to the 16 waves.
// SPREAD: slot s holds chunk big_pf_chunk(s); otherwise the copy is linear.
// live = 0 turns the copies into reads of the row's first KB (the last transform of a workgroup
// has nothing to prefetch, but a branch around the copies would make every wait for an
// earlier load a wait for all of them: the compiler merges the counts of both paths).
template <int PF, bool SPREAD>
__device__ __forceinline__ void big_prefetch(const float* src, float* dst, uint32_t t, uint32_t live)
{
    static_assert(PF % 2 == 0, "copies are dealt out in whole numbers per wave");
    const uint32_t w    = t >> 6;
    const uint32_t lane = t & 63u;
#pragma unroll
    for(int i = 0; i < PF / 2; ++i)
    {
        const uint32_t id    = w * (PF / 2) + i;
        const uint32_t slot  = id >> 3;
        const uint32_t part  = id & 7u;
        const uint32_t chunk = SPREAD ? 4u * (slot >> 1) + (slot & 1u) : slot;
        __builtin_amdgcn_global_load_lds((big_gptr)(src + live * (2048u * chunk + 256u * part) + 4u * lane),
                                         (big_lptr)(dst + 2048u * slot + 256u * part), 16, 0, 0);
    }
}

// the register <-> LDS transposition between two passes, one scalar plane at a time:
// slot s of thread t goes to wbase + WSTEP * big_slot_index(s), slot k comes from rbase + 1056 k
template <int WSTEP>
__device__ __forceinline__ void big_exchange(float2* r, float* lds, uint32_t wbase, uint32_t rbase)
{
#pragma unroll
    for(int s = 0; s < BIG_EPT; ++s)
        lds[wbase + WSTEP * big_slot_index(s)] = r[s].x;
    big_lds_barrier();
#pragma unroll
    for(int k = 0; k < BIG_EPT; ++k)
        r[k].x = lds[rbase + 1056 * k];
    big_lds_barrier();
#pragma unroll
    for(int s = 0; s < BIG_EPT; ++s)
        lds[wbase + WSTEP * big_slot_index(s)] = r[s].y;
    big_lds_barrier();
#pragma unroll
    for(int k = 0; k < BIG_EPT; ++k)
        r[k].y = lds[rbase + 1056 * k];
}

template <int MODE>
struct BigStream
{
    // chunks prefetched, first float of the prefetch area, dynamic LDS bytes
    static constexpr int    PF      = MODE == 1 ? 12 : 16;
    static constexpr int    PF_BASE = MODE == 1 ? 16384 : 0;
    static constexpr size_t LDS     = MODE == 1 ? 160 * 1024 : (size_t)(BIG_L + BIG_L / 32 + 32) * sizeof(float);
    // values per thread that come straight from global memory into registers
    static constexpr int ND = MODE == 2 ? 16 : 32 - PF;
};

// the chunks that are not prefetched, in rising order (complex and real forward transforms)
template <int PF>
struct BigDirectChunks
{
    int v[BIG_EPT];
    constexpr BigDirectChunks()
        : v()
    {
        int n = 0;
        for(int k = 0; k < BIG_EPT; ++k)
            if(!big_chunk_prefetched(k, PF))
                v[n++] = k;
    }
};

// MODE 0 complex (INV: inverse = re/im exchanged around the forward code), 1 real forward,
// 2 real inverse.  Rows must be 8-byte aligned; for MODE 0 and 1 input rows 16-byte aligned.
//
// One iteration of the loop, for transform i of this workgroup:
//   barrier; request the direct part of i; registers <- LDS (prefetched part of i), pass 0
//   starts on it; exchange; pass 1; exchange;
//   request the copy global -> LDS of the prefetched part of i + 1; pass 2;
//   wait for that copy; stores of i.
// Measured on MI355X and not kept: requesting the direct part of i + 1 between the stores of i
// (slower: loads queue behind the stores) or ahead of them (no change), nontemporal loads and
// stores (no gain; slower for the 8-byte aligned rows of 32769 bins, whose partial lines no
// longer merge in L2).
template <int MODE, bool INV>
__global__ __launch_bounds__(BIG_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void big32k_stream_kernel(
    const big_params p, const uint32_t total)
{
    extern __shared__ float lds[];
    float2*                 lds2 = reinterpret_cast<float2*>(lds);
    const float2*           tw   = static_cast<const float2*>(p.tw);
    constexpr bool          inv  = MODE == 2 || INV;
    constexpr int           HALF = BIG_L / 2;
    constexpr int           PF   = BigStream<MODE>::PF;
    constexpr int           ND   = BigStream<MODE>::ND;
    float*                  pf   = lds + BigStream<MODE>::PF_BASE;
    float2*                 pf2  = reinterpret_cast<float2*>(pf);
    constexpr BigDirectChunks<PF> direct_chunks;

    auto in_row = [&](uint32_t b) {
        const uint32_t l0 = b % p.lines[0];
        b /= p.lines[0];
        return static_cast<const float*>(p.in) + l0 * p.in_line[0] + (b % p.lines[1]) * p.in_line[1]
               + (b / p.lines[1]) * p.in_line[2];
    };
    auto out_row = [&](uint32_t b) {
        const uint32_t l0 = b % p.lines[0];
        b /= p.lines[0];
        return static_cast<float*>(p.out) + l0 * p.out_line[0] + (b % p.lines[1]) * p.out_line[1]
               + (b / p.lines[1]) * p.out_line[2];
    };
    // real inverse: rows of 32769 bins are 8-byte aligned only; the copy starts at the first
    // 16-byte aligned bin (0 or 1) and the LDS image is shifted by that much
    auto misalign = [](const float* row) { return (uint32_t)((reinterpret_cast<uintptr_t>(row) >> 3) & 1u); };
    auto prefetch = [&](const float* row, uint32_t t, uint32_t live) {
        if(MODE == 2)
            big_prefetch<PF, false>(row + 2 * misalign(row), pf, t, live);
        else
            big_prefetch<PF, true>(row, pf, t, live);
    };
    // direct value i of a row: the i-th chunk that is not prefetched, or for the real inverse
    // X_{L-j} of j = t + 1024 i (lanes run backwards)
    auto direct = [&](const float* row, uint32_t t, int i) {
        const float2* x = reinterpret_cast<const float2*>(row);
        if(MODE == 2)
            return (x + (BIG_L - 1024 * i - 1023))[1023u - t];
        return (x + 1024 * direct_chunks.v[i])[t];
    };
    // e^{-2 pi i t / 65536}: two registers that stay for the whole kernel
    float2 half_a = {0.0f, 0.0f};
    if(MODE != 0)
        half_a = static_cast<const float2*>(p.half_a)[threadIdx.x];

    uint32_t b = blockIdx.x;
    if(b >= total)
        return;
    prefetch(in_row(b), threadIdx.x, 1u);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    for(; b < total; b += gridDim.x)
    {
        // The thread index is re-read through an opaque copy in every iteration: the table
        // loads and LDS addresses below must not be hoisted out of the loop (62 registers of
        // loop-invariant twiddles would push the transform's own 64 registers into scratch).
        uint32_t t = threadIdx.x;
        asm volatile("" : "+v"(t));
        const uint32_t w1base = 33 * t;
        const uint32_t rbase  = t + (t >> 5);
        const uint32_t w2base = (t >> 5) * 1056 + (t & 31);
        float*         out    = out_row(b);
        const bool     more   = b + gridDim.x < total;
        const uint32_t live   = more ? 1u : 0u;
        const float*   next   = in_row(more ? b + gridDim.x : b);
        float2         r[BIG_EPT];
        // ---- the prefetched part is in LDS: every wave has waited for its own copies before its
        // last stores, here all waves meet
        big_lds_barrier();
        // the rest of the transform comes straight from global memory into registers
        const float* in = in_row(b);
        float2       nd[ND];
#pragma unroll
        for(int i = 0; i < ND; ++i)
            nd[i] = direct(in, t, i);
        float2 x0 = {0.0f, 0.0f}, xm = {0.0f, 0.0f}; // real inverse: bins 0 and L/2
        if(MODE == 2)
        {
            x0 = reinterpret_cast<const float2*>(in)[0];
            xm = reinterpret_cast<const float2*>(in)[HALF];
        }
        if(MODE != 2)
        {
#pragma unroll
            for(int s = 0; s < PF; ++s)
            {
                float2 v             = pf2[1024 * s + t];
                r[big_pf_chunk(s)] = inv ? c_swap(v) : v;
            }
#pragma unroll
            for(int i = 0; i < ND; ++i)
                r[direct_chunks.v[i]] = inv ? c_swap(nd[i]) : nd[i];
            big_lds_barrier();
        }
        else
        {
            // Hermitian bins -> half-length complex input.  The owner of j < L/2 forms z_j and
            // z_{L-j} from X_j (prefetched) and X_{L-j} (direct), keeps the first and hands the
            // second to its owner through LDS.  Only the real parts of bins 0 and L are used.
            const uint32_t mis = misalign(in);
            float2         xa[BIG_EPT / 2];
#pragma unroll
            for(int k = 0; k < BIG_EPT / 2; ++k)
                xa[k] = pf2[(int)(t + 1024 * k) - (int)(k == 0 && t == 0 ? 0u : mis)];
            if(t == 0)
                xa[0] = x0;
            float2 a = half_a; // opaque copy: its 16 products with the slot constants are not loop invariants to keep
            asm volatile("" : "+v"(a.x), "+v"(a.y));
            big_lds_barrier(); // every wave has read its prefetched bins: LDS is free for the hand-over
#pragma unroll
            for(int k = 0; k < BIG_EPT / 2; ++k)
            {
                const uint32_t j  = t + 1024 * k;
                const float2   xb = nd[k];
                float2         zj, zq;
                if(k == 0 && t == 0)
                {
                    zj.x = xa[k].x + xb.x;
                    zj.y = xa[k].x - xb.x;
                    r[k] = c_swap(zj);
                }
                else
                {
                    float2 tj = c_mul(a, big_w64(k));
                    float2 u, v;
                    u.x  = xa[k].x + xb.x;
                    u.y  = xa[k].y + xb.y;
                    v.x  = xa[k].x - xb.x;
                    v.y  = xa[k].y - xb.y;
                    zj.x = u.x + v.x * tj.y - u.y * tj.x;
                    zj.y = v.y + u.y * tj.y + v.x * tj.x;
                    zq.x = u.x - v.x * tj.y + u.y * tj.x;
                    zq.y = -v.y + u.y * tj.y + v.x * tj.x;
                    r[k] = c_swap(zj);
                    lds2[HALF - j] = c_swap(zq);
                }
            }
            if(t == 0)
            {
                float2 zm;
                zm.x    = 2.0f * xm.x;
                zm.y    = -2.0f * xm.y;
                lds2[0] = c_swap(zm);
            }
            big_lds_barrier();
#pragma unroll
            for(int k = BIG_EPT / 2; k < BIG_EPT; ++k)
                r[k] = lds2[t + 1024 * (k - BIG_EPT / 2)];
            big_lds_barrier();
        }

        Butterfly32<float>::run(r);
        big_exchange<1>(r, lds, w1base, rbase);
        big_twiddle(r, tw, 32u, t & 31u);
        Butterfly32<float>::run(r);
        // The tables of the last pass are requested before the exchange and have arrived after it:
        // loads return in order, so nothing may wait for a table entry once the copy of the next
        // transform is under way.
        BigTwiddle<float2> w2;
        w2.load(tw + 31 * 32, 1024u, t);
        big_lds_barrier();
        big_exchange<33>(r, lds, w2base, rbase);
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): the table entries
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        // ---- LDS is done with this transform (but for the hand-over area of the real forward
        // transform): start copying the next one (the last transform of a workgroup copies
        // nothing useful, see big_prefetch)
        big_lds_barrier();
        prefetch(next, t, live);
        w2.apply(r);
        // slot s will hold Z[t + 1024 big_slot_index(s)] (re/im exchanged when inverse)

        if(MODE != 1)
        {
            Butterfly32<float>::stage_a(r);
            // The copy has to be complete before this wave meets the others at the top of the
            // loop; waiting here, before the stores, keeps the stores out of the wait.
            __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
#pragma unroll
            for(int k2 = 0; k2 < 8; ++k2)
            {
                Butterfly32<float>::stage_b(r, k2);
#pragma unroll
                for(int s = 4 * k2; s < 4 * k2 + 4; ++s)
                {
                    float2 v = inv ? c_swap(r[s]) : r[s];
                    if(p.use_scale)
                    {
                        v.x *= (float)p.scale;
                        v.y *= (float)p.scale;
                    }
                    (reinterpret_cast<float2*>(out) + 1024 * big_slot_index(s))[t] = v;
                }
            }
            continue;
        }
        Butterfly32<float>::run(r);
        // ---- real forward: the owner of j < L/2 fetches Z_{L-j} from its owner through LDS
        // (two rounds of 8192 values in the 64 KB below the prefetch area) and writes X_j, X_{L-j}
        float2 zq[BIG_EPT / 2];
#pragma unroll
        for(int round = 0; round < 2; ++round)
        {
            if(round)
                big_lds_barrier(); // the first round has been read
#pragma unroll
            for(int s = 0; s < BIG_EPT; ++s)
                if(big_slot_index(s) >= 16 + 8 * round && big_slot_index(s) < 24 + 8 * round)
                    lds2[t + 1024 * (big_slot_index(s) - 16 - 8 * round)] = r[s];
            big_lds_barrier();
            // Z_{L-j} sits at index L/2 - j of the upper half: round 0 holds indices [0, 8192)
#pragma unroll
            for(int k = 8 - 8 * round; k < 16 - 8 * round; ++k)
                zq[k] = lds2[(HALF - (int)(t + 1024 * k)) & 8191];
            if(round && t == 0)
                zq[8] = lds2[0]; // j = 8192 pairs with index 8192, the first of the second round
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): the copy of the next transform is complete
        float2 a = half_a; // opaque copy: its 16 products with the slot constants are not loop invariants to keep
        asm volatile("" : "+v"(a.x), "+v"(a.y));
        float2*        ho = reinterpret_cast<float2*>(out);
        const float    sc = p.use_scale ? (float)p.scale : 1.0f;
        const uint32_t tr = 1023u - t;
#pragma unroll
        for(int s = 0; s < BIG_EPT; ++s)
        {
            const int k = big_slot_index(s);
            if(k >= BIG_EPT / 2)
            {
                if(k == BIG_EPT / 2 && t == 0)
                {
                    // bin L/2 pairs with itself
                    float2 o;
                    o.x      = r[s].x * sc;
                    o.y      = -r[s].y * sc;
                    ho[HALF] = o;
                }
                continue;
            }
            float2 zp = r[s];
            float2 o0, o1;
            if(k == 0 && t == 0)
            {
                o0.x = zp.x + zp.y;
                o0.y = 0.0f;
                o1.x = zp.x - zp.y;
                o1.y = 0.0f;
            }
            else
            {
                float2 tj = c_mul(a, big_w64(k));
                float2 u, v;
                u.x  = 0.5f * (zp.x + zq[k].x);
                u.y  = 0.5f * (zp.y + zq[k].y);
                v.x  = 0.5f * (zp.x - zq[k].x);
                v.y  = 0.5f * (zp.y - zq[k].y);
                o0.x = u.x + v.x * tj.y + u.y * tj.x;
                o0.y = v.y + u.y * tj.y - v.x * tj.x;
                o1.x = u.x - v.x * tj.y - u.y * tj.x;
                o1.y = -v.y + u.y * tj.y - v.x * tj.x;
            }
            o0.x *= sc;
            o0.y *= sc;
            o1.x *= sc;
            o1.y *= sc;
            (ho + 1024 * k)[t]                   = o0;
            (ho + (BIG_L - 1024 * k - 1023))[tr] = o1;
        }
    }
}

constexpr size_t BIG_LDS_BYTES = (size_t)(BIG_L + BIG_L / 32 + 32) * sizeof(float);
constexpr int    BIG_MAX_DEVICES = 64;

template <int MODE>
int launch_big(const big_params& p, uint32_t grid, hipStream_t stream)
{
    auto               kernel = big32k_kernel<MODE>;
    static FftLdsLimit limit;
    if(int rc = limit.allow(kernel))
        return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(BIG_THREADS), BIG_LDS_BYTES, stream, p);
    return (int)hipGetLastError();
}

// compute units of a device, asked once
int big_compute_units(int dev)
{
    static std::atomic<int> units[BIG_MAX_DEVICES];
    if(dev < 0 || dev >= BIG_MAX_DEVICES)
        return 0;
    int n = units[dev].load(std::memory_order_acquire);
    if(n == 0)
    {
        if(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            return 0;
        units[dev].store(n, std::memory_order_release);
    }
    return n;
}

template <int MODE, bool INV>
int launch_big_stream(const big_params& p, uint32_t total, hipStream_t stream)
{
    auto               kernel = big32k_stream_kernel<MODE, INV>;
    static FftLdsLimit limit;
    if(int rc = limit.allow(kernel))
        return rc;
    int dev = 0;
    if(int rc = (int)hipGetDevice(&dev))
        return rc;
    const int units = big_compute_units(dev);
    if(units <= 0)
        return (int)hipErrorInvalidDevice;
    // One workgroup fills a compute unit.  When the transforms divide evenly among the units, one
    // workgroup per unit walks through its share (measured with settled clocks, 4096 transforms on
    // 256 units: real forward 0.451 ms against 0.475 ms with four workgroups per unit in the grid,
    // real inverse 0.487 against 0.493, complex 0.442 against 0.454; eight per unit 0.484 / 0.508).
    // Otherwise four per unit, so that the units that finish early take the remainder.
    const uint64_t per_unit = total % (uint32_t)units == 0 ? 1 : 4;
    const uint32_t grid     = std::min<uint64_t>(total, per_unit * (uint32_t)units);
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(BIG_THREADS), BigStream<MODE>::LDS, stream, p, total);
    return (int)hipGetLastError();
}

// the streaming kernel copies 16 bytes per lane from global memory to LDS: complex and real
// forward rows have to start on 16-byte boundaries (real inverse rows: 8, handled in the kernel)
bool big_stream_ok(const big_params& p)
{
    if(p.mode == 2)
        return true;
    if(reinterpret_cast<uintptr_t>(p.in) % 16)
        return false;
    for(int i = 0; i < 3; ++i)
        if(p.lines[i] > 1 && (p.in_line[i] % 4) != 0)
            return false;
    return true;
}

} // namespace

extern "C" int fftrt_has_big32k(void)
{
    return 1;
}

extern "C" int fftrt_launch_big32k(const struct fftk_big_params* q, void* stream)
{
    uint64_t grid = 1;
    for(int i = 0; i < 3; ++i)
        grid *= q->lines[i];
    if(grid == 0 || grid >= (1ull << 31))
        return (int)hipErrorInvalidValue;
    hipStream_t s = (hipStream_t)stream;
    if(big_stream_ok(*q))
    {
        switch(q->mode)
        {
        case 0:
            return q->dir > 0 ? launch_big_stream<0, true>(*q, (uint32_t)grid, s)
                              : launch_big_stream<0, false>(*q, (uint32_t)grid, s);
        case 1:
            return launch_big_stream<1, false>(*q, (uint32_t)grid, s);
        case 2:
            return launch_big_stream<2, false>(*q, (uint32_t)grid, s);
        default:
            return (int)hipErrorInvalidValue;
        }
    }
    switch(q->mode)
    {
    case 0:
        return launch_big<0>(*q, (uint32_t)grid, s);
    case 1:
        return launch_big<1>(*q, (uint32_t)grid, s);
    default:
        return (int)hipErrorInvalidValue;
    }
}
