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
#include <hip/hip_runtime.h>
#include <mutex>

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
    static __device__ __forceinline__ void run(C* r)
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
#pragma unroll
        for(int k2 = 0; k2 < 8; ++k2)
        {
            C z[4] = {r[0 + 4 * k2], r[1 + 4 * k2], r[2 + 4 * k2], r[3 + 4 * k2]};
            Butterfly<T, 4>::run(z);
            // X[8 k1 + k2] = z[k1] stays in slot k1 + 4 k2 (see big_slot_index)
            r[0 + 4 * k2] = z[0];
            r[1 + 4 * k2] = z[1];
            r[2 + 4 * k2] = z[2];
            r[3 + 4 * k2] = z[3];
        }
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
__device__ __forceinline__ void big_twiddle(C* r, const C* tw, uint32_t c, uint32_t bl)
{
    C lo[8];
#pragma unroll
    for(int k = 1; k < 8; ++k)
    {
        lo[k] = tw[(k - 1) * c + bl];
        r[k]  = c_mul(r[k], lo[k]);
    }
#pragma unroll
    for(int a = 1; a < 4; ++a)
    {
        const C hi   = tw[(8 * a - 1) * c + bl];
        r[8 * a]     = c_mul(r[8 * a], hi);
#pragma unroll
        for(int b = 1; b < 8; ++b)
            r[8 * a + b] = c_mul(r[8 * a + b], c_mul(hi, lo[b]));
    }
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
        const float2* hb = static_cast<const float2*>(p.half_b);
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
                float2 tj = c_mul(a, hb[k]);
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
    const float2* hb = static_cast<const float2*>(p.half_b);
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
            float2 tj = c_mul(a, hb[k]);
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

constexpr size_t BIG_LDS_BYTES = (size_t)(BIG_L + BIG_L / 32 + 32) * sizeof(float);

template <int MODE>
int launch_big(const big_params& p, uint32_t grid, hipStream_t stream)
{
    auto                  kernel = big32k_kernel<MODE>;
    static std::once_flag once[16];
    int                   dev = 0;
    (void)hipGetDevice(&dev);
    int rc = 0;
    std::call_once(once[dev & 15], [&]() {
        rc = (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    });
    if(rc)
        return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(BIG_THREADS), BIG_LDS_BYTES, stream, p);
    return (int)hipGetLastError();
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
    switch(q->mode)
    {
    case 0:
        return launch_big<0>(*q, (uint32_t)grid, s);
    case 1:
        return launch_big<1>(*q, (uint32_t)grid, s);
    case 2:
        return launch_big<2>(*q, (uint32_t)grid, s);
    default:
        return (int)hipErrorInvalidValue;
    }
}
