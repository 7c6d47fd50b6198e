/* TEST INFRASTRUCTURE: a client written in plain C99 against include/rocfft/rocfft.h, the way
 * the reference's samples use the library (clients/samples/rocfft/rocfft_example_complexcomplex.cpp,
 * rocfft_example_realcomplex.cpp: setup -> description -> plan -> execution info with a work
 * buffer -> execute -> destroy -> cleanup).  Built twice: against the emulated runtime, where
 * "device" pointers are host pointers (CLIENT_HOST_BUFFERS), and against the real library with
 * buffers from the HIP runtime's C API.  Prints "ok" and returns 0 when every check holds. */
#include <math.h>
#include <rocfft/rocfft.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#ifdef CLIENT_HOST_BUFFERS
static void* dev_alloc(size_t bytes)
{
    return malloc(bytes);
}
static void dev_free(void* p)
{
    free(p);
}
static void to_dev(void* d, const void* h, size_t bytes)
{
    memcpy(d, h, bytes);
}
static void to_host(void* h, const void* d, size_t bytes)
{
    memcpy(h, d, bytes);
}
#else
#include <hip/hip_runtime_api.h>
static void* dev_alloc(size_t bytes)
{
    void* p = NULL;
    if(hipMalloc(&p, bytes) != hipSuccess)
        return NULL;
    return p;
}
static void dev_free(void* p)
{
    (void)hipFree(p);
}
static void to_dev(void* d, const void* h, size_t bytes)
{
    (void)hipMemcpy(d, h, bytes, hipMemcpyHostToDevice);
}
static void to_host(void* h, const void* d, size_t bytes)
{
    (void)hipDeviceSynchronize();
    (void)hipMemcpy(h, d, bytes, hipMemcpyDeviceToHost);
}
#endif

#define CHECK(call)                                                        \
    do                                                                     \
    {                                                                      \
        rocfft_status st_ = (call);                                        \
        if(st_ != rocfft_status_success)                                   \
        {                                                                  \
            fprintf(stderr, "%s failed with status %d\n", #call, (int)st_); \
            return 1;                                                      \
        }                                                                  \
    } while(0)

/* runs one plan with a caller-supplied work buffer */
static int run(rocfft_plan plan, void* in, void* out)
{
    rocfft_execution_info info = NULL;
    size_t                work = 0;
    void*                 wbuf = NULL;
    void*                 ins[1];
    void*                 outs[1];
    ins[0]  = in;
    outs[0] = out;
    CHECK(rocfft_execution_info_create(&info));
    CHECK(rocfft_plan_get_work_buffer_size(plan, &work));
    if(work)
    {
        wbuf = dev_alloc(work);
        if(!wbuf)
            return 1;
        CHECK(rocfft_execution_info_set_work_buffer(info, wbuf, work));
    }
    CHECK(rocfft_execute(plan, ins, out ? outs : NULL, info));
    CHECK(rocfft_execution_info_destroy(info));
    if(wbuf)
    {
        float probe; /* waits for the device before the work buffer goes away */
        to_host(&probe, in, sizeof(probe));
        dev_free(wbuf);
    }
    return 0;
}

/* complex forward then inverse, in place, length n, batch 3: x -> n x; and a known spectrum */
static int complex_round_trip(size_t n)
{
    const size_t batch = 3, total = n * batch;
    float*       h     = (float*)malloc(total * 2 * sizeof(float));
    float*       g     = (float*)malloc(total * 2 * sizeof(float));
    void*        d     = dev_alloc(total * 2 * sizeof(float));
    rocfft_plan  fwd = NULL, inv = NULL;
    size_t       lengths[1];
    size_t       i, b;
    double       err = 0, k0 = 3;
    if(!h || !g || !d)
        return 1;
    lengths[0] = n;
    /* batch b holds (b+1) e^{2 pi i k0 j / n}: its spectrum is (b+1) n at bin k0 */
    for(b = 0; b < batch; ++b)
        for(i = 0; i < n; ++i)
        {
            double ph              = 2.0 * 3.14159265358979323846 * k0 * (double)i / (double)n;
            h[2 * (b * n + i)]     = (float)((double)(b + 1) * cos(ph));
            h[2 * (b * n + i) + 1] = (float)((double)(b + 1) * sin(ph));
        }
    to_dev(d, h, total * 2 * sizeof(float));
    CHECK(rocfft_plan_create(&fwd, rocfft_placement_inplace, rocfft_transform_type_complex_forward,
                             rocfft_precision_single, 1, lengths, batch, NULL));
    CHECK(rocfft_plan_create(&inv, rocfft_placement_inplace, rocfft_transform_type_complex_inverse,
                             rocfft_precision_single, 1, lengths, batch, NULL));
    if(run(fwd, d, NULL))
        return 1;
    to_host(g, d, total * 2 * sizeof(float));
    for(b = 0; b < batch; ++b)
        for(i = 0; i < n; ++i)
        {
            double want = (i == (size_t)k0) ? (double)(b + 1) * (double)n : 0.0;
            double dr = g[2 * (b * n + i)] - want, di = g[2 * (b * n + i) + 1];
            if(fabs(dr) > err)
                err = fabs(dr);
            if(fabs(di) > err)
                err = fabs(di);
        }
    if(err > 1e-4 * (double)n)
    {
        fprintf(stderr, "complex forward n=%lu: error %g\n", (unsigned long)n, err);
        return 1;
    }
    if(run(inv, d, NULL))
        return 1;
    to_host(g, d, total * 2 * sizeof(float));
    err = 0;
    for(i = 0; i < 2 * total; ++i)
        if(fabs(g[i] / (double)n - h[i]) > err)
            err = fabs(g[i] / (double)n - h[i]);
    if(err > 1e-4)
    {
        fprintf(stderr, "complex round trip n=%lu: error %g\n", (unsigned long)n, err);
        return 1;
    }
    CHECK(rocfft_plan_destroy(fwd));
    CHECK(rocfft_plan_destroy(inv));
    dev_free(d);
    free(h);
    free(g);
    return 0;
}

/* out-of-place real forward of a 2D array in double precision with a description (scale
 * factor and explicit layout), checked against the direct sum */
static int real_2d(size_t n0, size_t n1)
{
    const size_t           h0 = n0 / 2 + 1;
    double*                x  = (double*)malloc(n0 * n1 * sizeof(double));
    double*                y  = (double*)malloc(h0 * n1 * 2 * sizeof(double));
    void*                  dx = dev_alloc(n0 * n1 * sizeof(double));
    void*                  dy = dev_alloc(h0 * n1 * 2 * sizeof(double));
    rocfft_plan_description desc = NULL;
    rocfft_plan             plan = NULL;
    size_t                  lengths[2], istr[2], ostr[2], off[2] = {0, 0};
    size_t                  i, j, k0, k1;
    const double            scale = 0.5;
    double                  err = 0;
    if(!x || !y || !dx || !dy)
        return 1;
    lengths[0] = n0; /* fastest dimension first */
    lengths[1] = n1;
    istr[0]    = 1;
    istr[1]    = n0;
    ostr[0]    = 1;
    ostr[1]    = h0;
    for(i = 0; i < n0 * n1; ++i)
        x[i] = (double)((i * 7919u) % 1000u) / 1000.0 - 0.5;
    to_dev(dx, x, n0 * n1 * sizeof(double));
    CHECK(rocfft_plan_description_create(&desc));
    CHECK(rocfft_plan_description_set_data_layout(desc, rocfft_array_type_real,
                                                  rocfft_array_type_hermitian_interleaved, off, off, 2, istr,
                                                  n0 * n1, 2, ostr, h0 * n1));
    CHECK(rocfft_plan_description_set_scale_factor(desc, scale));
    CHECK(rocfft_plan_create(&plan, rocfft_placement_notinplace, rocfft_transform_type_real_forward,
                             rocfft_precision_double, 2, lengths, 1, desc));
    CHECK(rocfft_plan_description_destroy(desc)); /* the plan holds a copy */
    if(run(plan, dx, dy))
        return 1;
    to_host(y, dy, h0 * n1 * 2 * sizeof(double));
    for(k1 = 0; k1 < n1; ++k1)
        for(k0 = 0; k0 < h0; ++k0)
        {
            double re = 0, im = 0;
            for(j = 0; j < n1; ++j)
                for(i = 0; i < n0; ++i)
                {
                    double ph = -2.0 * 3.14159265358979323846
                                * ((double)(k0 * i % n0) / (double)n0 + (double)(k1 * j % n1) / (double)n1);
                    re += x[j * n0 + i] * cos(ph);
                    im += x[j * n0 + i] * sin(ph);
                }
            re *= scale;
            im *= scale;
            if(fabs(y[2 * (k1 * h0 + k0)] - re) > err)
                err = fabs(y[2 * (k1 * h0 + k0)] - re);
            if(fabs(y[2 * (k1 * h0 + k0) + 1] - im) > err)
                err = fabs(y[2 * (k1 * h0 + k0) + 1] - im);
        }
    if(err > 1e-10)
    {
        fprintf(stderr, "real 2D %lux%lu: error %g\n", (unsigned long)n0, (unsigned long)n1, err);
        return 1;
    }
    CHECK(rocfft_plan_destroy(plan));
    dev_free(dx);
    dev_free(dy);
    free(x);
    free(y);
    return 0;
}

int main(void)
{
    char version[64];
    CHECK(rocfft_setup());
    CHECK(rocfft_get_version_string(version, sizeof(version)));
    if(strlen(version) == 0)
        return 1;
    if(complex_round_trip(64) || complex_round_trip(1000) || complex_round_trip(97) || complex_round_trip(20000))
        return 1;
    if(real_2d(30, 12) || real_2d(17, 8))
        return 1;
    CHECK(rocfft_cleanup());
    printf("ok %s\n", version);
    return 0;
}
