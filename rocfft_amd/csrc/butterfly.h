// butterfly.h -- forward radix-R DFT butterflies on register arrays.
//
// Only the forward sign (e^{-2 pi i jk/R}) is implemented: inverse transforms
// run the same code on data whose real and imaginary parts are exchanged,
// because IDFT(x) = swap(DFT(swap(x))).
//
// The reference's equivalents are the FwdRadN functions under
// library/src/device/generator/rtc_radix_functions/ (radix_2.h .. radix_16.h);
// these are independent derivations from the DFT definition.
#ifndef ROCFFT_AMD_BUTTERFLY_H
#define ROCFFT_AMD_BUTTERFLY_H

#include <hip/hip_runtime.h>

template <typename T>
struct cplx_of;
template <>
struct cplx_of<float>
{
    typedef float2 type;
};
template <>
struct cplx_of<double>
{
    typedef double2 type;
};

#define FFT_DEV __host__ __device__ __forceinline__

template <typename C>
FFT_DEV C c_add(C a, C b)
{
    C r;
    r.x = a.x + b.x;
    r.y = a.y + b.y;
    return r;
}
template <typename C>
FFT_DEV C c_sub(C a, C b)
{
    C r;
    r.x = a.x - b.x;
    r.y = a.y - b.y;
    return r;
}
template <typename C>
FFT_DEV C c_mul(C a, C b)
{
    C r;
    r.x = a.x * b.x - a.y * b.y;
    r.y = a.x * b.y + a.y * b.x;
    return r;
}
// a * conj(b)
template <typename C>
FFT_DEV C c_mulc(C a, C b)
{
    C r;
    r.x = a.x * b.x + a.y * b.y;
    r.y = a.y * b.x - a.x * b.y;
    return r;
}
// multiply by -i
template <typename C>
FFT_DEV C c_mnegi(C a)
{
    C r;
    r.x = a.y;
    r.y = -a.x;
    return r;
}
template <typename C>
FFT_DEV C c_swap(C a)
{
    C r;
    r.x = a.y;
    r.y = a.x;
    return r;
}

template <typename T, int R>
struct Butterfly;

template <typename T>
struct Butterfly<T, 2>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        C a = c_add(r[0], r[1]);
        C b = c_sub(r[0], r[1]);
        r[0] = a;
        r[1] = b;
    }
};

template <typename T>
struct Butterfly<T, 3>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T s = (T)0.866025403784438646763723170752936183; // sin(2 pi/3)
        C       a = c_add(r[1], r[2]);
        C       b = c_sub(r[1], r[2]);
        C       t;
        t.x = r[0].x - (T)0.5 * a.x;
        t.y = r[0].y - (T)0.5 * a.y;
        // -i * s * b
        C u;
        u.x  = s * b.y;
        u.y  = -s * b.x;
        r[0] = c_add(r[0], a);
        r[1] = c_add(t, u);
        r[2] = c_sub(t, u);
    }
};

template <typename T>
struct Butterfly<T, 4>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        C t0 = c_add(r[0], r[2]);
        C t1 = c_sub(r[0], r[2]);
        C t2 = c_add(r[1], r[3]);
        C t3 = c_mnegi(c_sub(r[1], r[3]));
        r[0] = c_add(t0, t2);
        r[1] = c_add(t1, t3);
        r[2] = c_sub(t0, t2);
        r[3] = c_sub(t1, t3);
    }
};

// odd prime radix by the symmetric/antisymmetric split:
//   a_m = r_m + r_{R-m}, b_m = r_m - r_{R-m},
//   X_k, X_{R-k} = (r_0 + sum_m cos(2 pi km/R) a_m) -/+ i (sum_m sin(2 pi km/R) b_m)
template <typename T, int R>
struct OddButterfly
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r, const T* cs, const T* sn)
    {
        constexpr int H = (R - 1) / 2;
        C             a[H], b[H];
#pragma unroll
        for(int m = 0; m < H; ++m)
        {
            a[m] = c_add(r[m + 1], r[R - 1 - m]);
            b[m] = c_sub(r[m + 1], r[R - 1 - m]);
        }
        C x0 = r[0];
        C s0 = r[0];
#pragma unroll
        for(int m = 0; m < H; ++m)
            s0 = c_add(s0, a[m]);
        r[0] = s0;
#pragma unroll
        for(int k = 1; k <= H; ++k)
        {
            C t = x0;
            C u;
            u.x = 0;
            u.y = 0;
#pragma unroll
            for(int m = 1; m <= H; ++m)
            {
                int idx = (k * m) % R; // table index, compile-time after unrolling
                t.x += cs[idx] * a[m - 1].x;
                t.y += cs[idx] * a[m - 1].y;
                u.x += sn[idx] * b[m - 1].x;
                u.y += sn[idx] * b[m - 1].y;
            }
            // X_k = t - i u ; X_{R-k} = t + i u
            r[k].x     = t.x + u.y;
            r[k].y     = t.y - u.x;
            r[R - k].x = t.x - u.y;
            r[R - k].y = t.y + u.x;
        }
    }
};

template <typename T>
struct Butterfly<T, 5>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T cs[5] = {(T)1.0,
                         (T)0.309016994374947424102293417182819059,
                         (T)-0.809016994374947424102293417182819059,
                         (T)-0.809016994374947424102293417182819059,
                         (T)0.309016994374947424102293417182819059};
        const T sn[5] = {(T)0.0,
                         (T)0.951056516295153572116439333379382143,
                         (T)0.587785252292473129168705954639072769,
                         (T)-0.587785252292473129168705954639072769,
                         (T)-0.951056516295153572116439333379382143};
        OddButterfly<T, 5>::run(r, cs, sn);
    }
};

template <typename T>
struct Butterfly<T, 7>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T cs[7] = {(T)1.0,
                         (T)0.623489801858733530525004884004239811,
                         (T)-0.222520933956314404288902564496794760,
                         (T)-0.900968867902419126236102319507445051,
                         (T)-0.900968867902419126236102319507445051,
                         (T)-0.222520933956314404288902564496794760,
                         (T)0.623489801858733530525004884004239811};
        const T sn[7] = {(T)0.0,
                         (T)0.781831482468029808708444526674057750,
                         (T)0.974927912181823607018131682993931217,
                         (T)0.433883739117558120475768332848358754,
                         (T)-0.433883739117558120475768332848358754,
                         (T)-0.974927912181823607018131682993931217,
                         (T)-0.781831482468029808708444526674057750};
        OddButterfly<T, 7>::run(r, cs, sn);
    }
};

template <typename T>
struct Butterfly<T, 11>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T cs[11] = {(T)1.0,
                          (T)0.841253532831181168861811648919367718,
                          (T)0.415415013001886425529274149229623203,
                          (T)-0.142314838273285140443792668616369669,
                          (T)-0.654860733945285064056925072466293553,
                          (T)-0.959492973614497389890368057066327700,
                          (T)-0.959492973614497389890368057066327700,
                          (T)-0.654860733945285064056925072466293553,
                          (T)-0.142314838273285140443792668616369669,
                          (T)0.415415013001886425529274149229623203,
                          (T)0.841253532831181168861811648919367718};
        const T sn[11] = {(T)0.0,
                          (T)0.540640817455597582107635954318691696,
                          (T)0.909631995354518371411715383079028460,
                          (T)0.989821441880932732376092037776718787,
                          (T)0.755749574354258283774035843972344420,
                          (T)0.281732556841429697711417047245708656,
                          (T)-0.281732556841429697711417047245708656,
                          (T)-0.755749574354258283774035843972344420,
                          (T)-0.989821441880932732376092037776718787,
                          (T)-0.909631995354518371411715383079028460,
                          (T)-0.540640817455597582107635954318691696};
        OddButterfly<T, 11>::run(r, cs, sn);
    }
};

template <typename T>
struct Butterfly<T, 13>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T cs[13] = {(T)1.0,
                          (T)0.885456025653209896603457178692860172,
                          (T)0.568064746731155802170125129211003647,
                          (T)0.120536680255323001959974834154866815,
                          (T)-0.354604887042535625312577614632482588,
                          (T)-0.748510748171101098340318217213128354,
                          (T)-0.970941817426052027133653644877719690,
                          (T)-0.970941817426052027133653644877719690,
                          (T)-0.748510748171101098340318217213128354,
                          (T)-0.354604887042535625312577614632482588,
                          (T)0.120536680255323001959974834154866815,
                          (T)0.568064746731155802170125129211003647,
                          (T)0.885456025653209896603457178692860172};
        const T sn[13] = {(T)0.0,
                          (T)0.464723172043768545964430247174500899,
                          (T)0.822983865893656386660032296954293963,
                          (T)0.992708874098054008658010731471478137,
                          (T)0.935016242685414800802188714521834425,
                          (T)0.663122658240795273726928868884563733,
                          (T)0.239315664287557679995803516167874459,
                          (T)-0.239315664287557679995803516167874459,
                          (T)-0.663122658240795273726928868884563733,
                          (T)-0.935016242685414800802188714521834425,
                          (T)-0.992708874098054008658010731471478137,
                          (T)-0.822983865893656386660032296954293963,
                          (T)-0.464723172043768545964430247174500899};
        OddButterfly<T, 13>::run(r, cs, sn);
    }
};

template <typename T>
struct Butterfly<T, 17>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T cs[17] = {(T)1.0,
                          (T)9.32472229404355804573115891821563386e-1,
                          (T)7.39008917220659115924534309872648106e-1,
                          (T)4.45738355776538267396457549379486855e-1,
                          (T)9.22683594633019952396511071545064804e-2,
                          (T)-2.73662990072082863539077935436813432e-1,
                          (T)-6.02634636379256389178588154986840622e-1,
                          (T)-8.50217135729614152134143922949352058e-1,
                          (T)-9.82973099683901778281948844855198716e-1,
                          (T)-9.82973099683901778281948844855198716e-1,
                          (T)-8.50217135729614152134143922949352058e-1,
                          (T)-6.02634636379256389178588154986840622e-1,
                          (T)-2.73662990072082863539077935436813432e-1,
                          (T)9.22683594633019952396511071545064804e-2,
                          (T)4.45738355776538267396457549379486855e-1,
                          (T)7.39008917220659115924534309872648106e-1,
                          (T)9.32472229404355804573115891821563386e-1};
        const T sn[17] = {(T)0.0,
                          (T)3.61241666187152948744714596183700164e-1,
                          (T)6.73695643646557211712691912425694616e-1,
                          (T)8.95163291355062322067016499753785457e-1,
                          (T)9.95734176295034521871191178905481784e-1,
                          (T)9.61825643172819070408796290731518550e-1,
                          (T)7.98017227280239503332805112796261369e-1,
                          (T)5.26432162877355800244607799140699566e-1,
                          (T)1.83749517816570331574408839620727582e-1,
                          (T)-1.83749517816570331574408839620727582e-1,
                          (T)-5.26432162877355800244607799140699566e-1,
                          (T)-7.98017227280239503332805112796261369e-1,
                          (T)-9.61825643172819070408796290731518550e-1,
                          (T)-9.95734176295034521871191178905481784e-1,
                          (T)-8.95163291355062322067016499753785457e-1,
                          (T)-6.73695643646557211712691912425694616e-1,
                          (T)-3.61241666187152948744714596183700164e-1};
        OddButterfly<T, 17>::run(r, cs, sn);
    }
};

template <typename T>
struct Butterfly<T, 8>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T h = (T)0.707106781186547524400844362104849039; // 1/sqrt(2)
        C       e[4] = {r[0], r[2], r[4], r[6]};
        C       o[4] = {r[1], r[3], r[5], r[7]};
        Butterfly<T, 4>::run(e);
        Butterfly<T, 4>::run(o);
        // o[k] *= W_8^k
        C t;
        t.x  = h * (o[1].x + o[1].y);
        t.y  = h * (o[1].y - o[1].x);
        o[1] = t;
        o[2] = c_mnegi(o[2]);
        t.x  = h * (o[3].y - o[3].x);
        t.y  = -h * (o[3].x + o[3].y);
        o[3] = t;
#pragma unroll
        for(int k = 0; k < 4; ++k)
        {
            r[k]     = c_add(e[k], o[k]);
            r[k + 4] = c_sub(e[k], o[k]);
        }
    }
};

template <typename T>
struct Butterfly<T, 16>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        // n = n1 + 4 n2, k = 4 k1 + k2:
        //   y[n1][k2] = sum_n2 x[n1 + 4 n2] W_4^{n2 k2}
        //   X[4 k1 + k2] = sum_n1 W_4^{n1 k1} (W_16^{n1 k2} y[n1][k2])
        const T c1 = (T)0.923879532511286756128183189396788287; // cos(pi/8)
        const T s1 = (T)0.382683432365089771728459984030398866; // sin(pi/8)
        const T h  = (T)0.707106781186547524400844362104849039;
        C       y[4][4];
#pragma unroll
        for(int n1 = 0; n1 < 4; ++n1)
        {
            y[n1][0] = r[n1];
            y[n1][1] = r[n1 + 4];
            y[n1][2] = r[n1 + 8];
            y[n1][3] = r[n1 + 12];
            Butterfly<T, 4>::run(y[n1]);
        }
        // W_16^m = (cos(m pi/8), -sin(m pi/8)), m = n1*k2 in {1,2,3,4,6,9}
        const C w1 = {c1, -s1};
        const C w2 = {h, -h};
        const C w3 = {s1, -c1};
        const C w6 = {-h, -h};
        const C w9 = {-c1, s1};
        y[1][1]    = c_mul(y[1][1], w1);
        y[1][2]    = c_mul(y[1][2], w2);
        y[1][3]    = c_mul(y[1][3], w3);
        y[2][1]    = c_mul(y[2][1], w2);
        y[2][2]    = c_mnegi(y[2][2]);
        y[2][3]    = c_mul(y[2][3], w6);
        y[3][1]    = c_mul(y[3][1], w3);
        y[3][2]    = c_mul(y[3][2], w6);
        y[3][3]    = c_mul(y[3][3], w9);
#pragma unroll
        for(int k2 = 0; k2 < 4; ++k2)
        {
            C z[4] = {y[0][k2], y[1][k2], y[2][k2], y[3][k2]};
            Butterfly<T, 4>::run(z);
            r[k2]      = z[0];
            r[4 + k2]  = z[1];
            r[8 + k2]  = z[2];
            r[12 + k2] = z[3];
        }
    }
};

// Composite radix R = A*B from two smaller butterflies (Cooley-Tukey with n = B a + b,
// k = k1 + A k2):
//   y[b][k1]      = sum_a x[B a + b] W_A^{a k1}
//   X[k1 + A k2]  = sum_b W_B^{b k2} (W_R^{b k1} y[b][k1])
// cs[m], sn[m] = cos, sin(2 pi m / R); the table indices are compile-time after unrolling.
template <typename T, int A, int B>
struct CompositeButterfly
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r, const T* cs, const T* sn)
    {
        constexpr int R = A * B;
        C             y[B][A];
#pragma unroll
        for(int b = 0; b < B; ++b)
        {
#pragma unroll
            for(int a = 0; a < A; ++a)
                y[b][a] = r[B * a + b];
            Butterfly<T, A>::run(y[b]);
        }
#pragma unroll
        for(int b = 1; b < B; ++b)
#pragma unroll
            for(int k1 = 1; k1 < A; ++k1)
            {
                const int m = (b * k1) % R;
                C         w;
                w.x      = cs[m];
                w.y      = -sn[m];
                y[b][k1] = c_mul(y[b][k1], w);
            }
#pragma unroll
        for(int k1 = 0; k1 < A; ++k1)
        {
            C z[B];
#pragma unroll
            for(int b = 0; b < B; ++b)
                z[b] = y[b][k1];
            Butterfly<T, B>::run(z);
#pragma unroll
            for(int k2 = 0; k2 < B; ++k2)
                r[k1 + A * k2] = z[k2];
        }
    }
};

template <typename T>
struct Butterfly<T, 6>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T cs[6] = {(T)1.0,
                         (T)0.5,
                         (T)-0.5,
                         (T)-1.0,
                         (T)-0.5,
                         (T)0.5};
        const T sn[6] = {(T)0.0,
                         (T)0.866025403784438646763723170752936183,
                         (T)0.866025403784438646763723170752936183,
                         (T)4.13406421965279764729938061032096894e-43,
                         (T)-0.866025403784438646763723170752936183,
                         (T)-0.866025403784438646763723170752936183};
        CompositeButterfly<T, 3, 2>::run(r, cs, sn);
    }
};

template <typename T>
struct Butterfly<T, 9>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T cs[9] = {(T)1.0,
                         (T)0.766044443118978035202392650555416674,
                         (T)0.173648177666930348851716626769314796,
                         (T)-0.5,
                         (T)-0.93969262078590838405410927732473147,
                         (T)-0.93969262078590838405410927732473147,
                         (T)-0.5,
                         (T)0.173648177666930348851716626769314796,
                         (T)0.766044443118978035202392650555416674};
        const T sn[9] = {(T)0.0,
                         (T)0.642787609686539326322643409907263433,
                         (T)0.984807753012208059366743024589523014,
                         (T)0.866025403784438646763723170752936183,
                         (T)0.342020143325668733044099614682259581,
                         (T)-0.342020143325668733044099614682259581,
                         (T)-0.866025403784438646763723170752936183,
                         (T)-0.984807753012208059366743024589523014,
                         (T)-0.642787609686539326322643409907263433};
        CompositeButterfly<T, 3, 3>::run(r, cs, sn);
    }
};

template <typename T>
struct Butterfly<T, 10>
{
    typedef typename cplx_of<T>::type C;
    static FFT_DEV void               run(C* r)
    {
        const T cs[10] = {(T)1.0,
                          (T)0.809016994374947424102293417182819059,
                          (T)0.309016994374947424102293417182819059,
                          (T)-0.309016994374947424102293417182819059,
                          (T)-0.809016994374947424102293417182819059,
                          (T)-1.0,
                          (T)-0.809016994374947424102293417182819059,
                          (T)-0.309016994374947424102293417182819059,
                          (T)0.309016994374947424102293417182819059,
                          (T)0.809016994374947424102293417182819059};
        const T sn[10] = {(T)0.0,
                          (T)0.587785252292473129168705954639072769,
                          (T)0.951056516295153572116439333379382143,
                          (T)0.951056516295153572116439333379382143,
                          (T)0.587785252292473129168705954639072769,
                          (T)4.13406421965279764729938061032096894e-43,
                          (T)-0.587785252292473129168705954639072769,
                          (T)-0.951056516295153572116439333379382143,
                          (T)-0.951056516295153572116439333379382143,
                          (T)-0.587785252292473129168705954639072769};
        CompositeButterfly<T, 5, 2>::run(r, cs, sn);
    }
};

#endif
