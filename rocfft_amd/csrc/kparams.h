// kparams.h -- launch descriptors shared by the host planner and the device kernels.
//
// One "tile pass" is a batch of 1D FFTs of length n.  A workgroup owns a tile of
// W transforms that are neighbours along the "tile" dimension, stages the tile in
// LDS, runs every Stockham pass there and writes the tile back.  Whether global
// accesses run fastest along the transform or along the tile dimension is chosen
// per side, so the same kernel serves unit-stride rows, strided columns and
// row-in/column-out (transposing) passes.
#ifndef ROCFFT_AMD_KPARAMS_H
#define ROCFFT_AMD_KPARAMS_H

#include <stdint.h>

#define FFTK_MAX_PASSES 12
#define FFTK_REG_ELEMS 17 // complex values a thread keeps in registers per pass (one radix-17 butterfly)

// how a tile element is fetched
enum fftk_load_op
{
    FFTK_LOAD_COMPLEX     = 0, // (re, im) from in0/in1
    FFTK_LOAD_REAL        = 1, // re from in0, im = 0
    FFTK_LOAD_C2R_PRE     = 2, // Hermitian bins -> half-length complex input of the inverse FFT
    FFTK_LOAD_HERM_EXPAND = 3  // bins 0..n_in/2 plus their conjugate mirror (odd-length real inverse)
};

// how a tile element is written
enum fftk_store_op
{
    FFTK_STORE_COMPLEX  = 0,
    FFTK_STORE_REAL     = 1, // real part only, to out0
    FFTK_STORE_R2C_POST = 2  // half-length complex spectrum -> n+1 Hermitian bins
};

enum fftk_flags
{
    FFTK_F_TWIDDLE_STORE = 1 << 0, // multiply output (j, q) by W_L^{j*q}
    FFTK_F_CHIRP_LOAD    = 1 << 1, // multiply input by conj(chirp[idx]), zero beyond blu_n
    FFTK_F_CHIRP_STORE   = 1 << 2, // multiply output by conj(chirp[idx]), skip beyond blu_n
    FFTK_F_CONV          = 1 << 3, // forward FFT, multiply by convb, inverse FFT
    FFTK_F_SCALE         = 1 << 4, // multiply output by scale
    FFTK_F_CHIRP_CONJ    = 1 << 5  // use the conjugate chirp (inverse-direction Bluestein)
};

// User load/store callbacks of an execution (reference library/include/rocfft/rocfft.h:533-612),
// called from inside the first and the last kernel of a plan:
//   T    load_cb (T* data, size_t offset, void* cbdata, void* sharedMem);
//   void store_cb(T* data, size_t offset, T element, void* cbdata, void* sharedMem);
// data is the buffer pointer given to rocfft_execute, offset counts elements of the array's type
// (real scalars, or complex pairs for interleaved complex arrays).  The kernels address scalars
// relative to their own base pointers; *_off is the distance of that base from the user's
// pointer, in scalars.  A null function pointer means plain memory access.
struct fftk_cb
{
    const void* load_fn;
    void*       load_data;
    const void* in_base;    // the user's input pointer
    int64_t     in_off;     // scalars from in_base to the kernel's input base
    uint32_t    in_complex; // 1: the callback's element is a complex pair
    uint32_t    out_complex;
    const void* store_fn;
    void*       store_data;
    void*       out_base;
    int64_t     out_off;
};

struct fftk_params
{
    // The members the compiled kernels read on every path come first and close together: a
    // kernel fetches its arguments from memory 64 bytes at a time, and a workgroup that runs
    // alone (a small transform) waits for each such fetch.
    // buffers (filled in at execute)
    const void* in0;
    const void* in1;
    void*       out0;
    void*       out1;
    const void* tw; // stacked per-pass twiddles
    uint32_t flags;
    int32_t  dir; // -1 forward, +1 inverse
    uint32_t load_op, store_op;
    // work split
    uint32_t W;        // transforms per workgroup (power of two)
    uint32_t wshift;   // log2(W)
    uint32_t wfast;    // compute phase: 1 = neighbouring lanes take neighbouring transforms
    uint32_t nthreads;
    uint32_t grid;       // number of workgroups
    uint32_t xcd_remap;  // renumber workgroups so that each XCD gets a contiguous range of tiles
    uint32_t oc0_first;  // outer axis 0 runs faster than the tile index in the workgroup numbering
    uint32_t direct_in;  // fast kernel: first pass loads global memory straight into registers
    uint32_t direct_out; // fast kernel: last pass stores straight from registers
    uint32_t stage_io; // lean path: move the tile between global memory and LDS with consecutive
                       // lanes on consecutive elements (transforms too short for coalesced
                       // register loads)
    uint32_t t_is_c, t_os_c, w_is_c, w_os_c;
    uint32_t in_planar, out_planar; // lean path: that side is a planar complex array (real parts
                                    // at in0/out0, imaginary parts at in1/out1)
    uint32_t in_nt, out_nt;     // lean path, interleaved arrays: access that side with the nontemporal hint
    uint32_t in_half, out_half; // lean path, single precision: that side is an array of IEEE half
                                // pairs (in0 / out0 point at half values, strides and offsets count
                                // half scalars)
    // Folded tile axis (w_inner != 0): tile index g counts (i, b) pairs, i = g % w_inner along the
    // short contiguous axis (strides w_is / w_os) and b = g / w_inner along a second axis (strides
    // w2_is / w2_os: the transforms of a batch).  A column pass over very short rows then still
    // fills its workgroups.  tile_cnt is the number of pairs.
    uint32_t w_inner;
    uint32_t w2_is_c, w2_os_c; // lean path: w2_is / w2_os in elements
    // index space: transform, tile dimension, three outer dimensions; strides in scalars
    uint32_t tile_cnt;
    uint32_t oc[3];
    uint32_t aux_dim;   // which index is q: 0 none, 1 tile, 2/3/4 outer 0/1/2
    uint32_t aux_shift; // aux_dim 1: q = tile index >> aux_shift (a faster plain axis was merged into the tile axis)
    int64_t  w_is, w_os, o_is[3], o_os[3], t_is, t_os, w2_is, w2_os;
    double   scale;
    uint32_t n_in;  // input elements j >= n_in read as zero
    uint32_t n_out; // output elements j >= n_out are not written
    // tables of the fused operations
    const void* ltw;       // two-level table for W_L^u: lo[0 .. 1<<ltw_shift), then hi[]
    const void* half_tw;   // e^{-2 pi i j/(2n)}, j in [0, n/2], for the real pre/post steps
    const void* chirp;     // Bluestein chirp e^{+i pi m^2/N}, m in [0, blu_n)
    const void* convb;     // spectrum the tile is multiplied with in CONV mode
    const void* tw2;       // fused 2D kernel: stacked twiddles of the second dimension
    uint32_t    ltw_shift; //
    uint32_t    ltw_qmul, ltw_qadd; // the large twiddle of output j is W_L^{j (q ltw_qmul + ltw_qadd)}
    uint32_t    blu_n;
    uint32_t    chirp_js, chirp_qs; // logical sample index = j*chirp_js + q*chirp_qs
    uint32_t    convb_qs;           // convb index = j + q*convb_qs
    uint32_t    n2;    // fused 2D kernel: length of the second (strided) dimension
    uint32_t    fast;  // 1 = a kernel with this exact pass schedule is compiled in: use it
    uint32_t    lean;  // fast kernel: complex arrays on both sides, strides in
                       // complex elements fit 32 bits: branch-free addressing path
    // transform: the schedule of the run-time-schedule kernel
    uint32_t n;                      // FFT length
    uint32_t nf;                     // number of passes
    uint32_t T;        // threads per transform
    uint32_t pitch;    // LDS elements between transforms of a tile
    uint32_t padshift; // LDS index i is stored at i + (i >> padshift)
    uint32_t in_fast_tile, out_fast_tile; // global access runs fastest along the tile dimension
    uint32_t radix[FFTK_MAX_PASSES]; // radix of each pass
    uint32_t cum[FFTK_MAX_PASSES];   // product of the radices before the pass
    uint32_t cshift[FFTK_MAX_PASSES]; // log2(cum) when cum is a power of two, else 0xff
    uint32_t twoff[FFTK_MAX_PASSES]; // offset of the pass in the stacked twiddle table
    struct fftk_cb cb; // run-time-schedule kernel only
};

// standalone even-length real post-/pre-processing over natural-order rows
struct fftk_real_params
{
    uint32_t    half; // complex length L (the real length is 2L)
    uint32_t    rows0, rows1, rows2; // three row dimensions
    int64_t     z_s, z_r0, z_r1, z_r2; // complex side: element stride and row strides, in scalars
    int64_t     h_s, h_r0, h_r1, h_r2; // Hermitian side
    const void* z0;
    const void* z1;
    void*       zo0;
    void*       zo1;
    const void* h0;
    const void* h1;
    void*       ho0;
    void*       ho1;
    const void* half_tw; // e^{-2 pi i j/(2L)}, j in [0, L/2]
    double      scale;
    uint32_t    use_scale;
    struct fftk_cb cb; // post: store side (Hermitian bins); pre: load side
};

// element-wise row copy between array kinds: real -> complex, complex -> real, Hermitian half
// -> full conjugate-symmetric row, complex row -> its first elements.  The slow path of
// odd-length real transforms too long for one kernel runs a complex transform between two
// of these.
struct fftk_copy_params
{
    uint32_t    cnt;         // elements written per row
    uint32_t    mirror_from; // source index j >= mirror_from reads element mirror_n - j, conjugated
    uint32_t    mirror_n;    //   (mirror_from = 0: no mirroring)
    uint32_t    src_real;    // the source holds real values (imaginary part reads as zero)
    uint32_t    dst_real;    // only the real part is written
    uint32_t    zero_im0;    // the imaginary part of source element 0 reads as zero
    uint32_t    rows0, rows1, rows2;
    int64_t     s_s, s_r0, s_r1, s_r2; // source element stride and row strides, in scalars
    int64_t     d_s, d_r0, d_r1, d_r2;
    const void* s0; // real parts
    const void* s1; // imaginary parts
    void*       d0;
    void*       d1;
    double      scale;
    uint32_t    use_scale;
    struct fftk_cb cb;
};

// Copy of every element of a transform's input (or output) between the user's buffer and a
// scratch buffer with the same layout, through the user's load (or store) callback:
//   T load_cb(T* data, size_t offset, void* cbdata, void* sharedMem);
//   void store_cb(T* data, size_t offset, T element, void* cbdata, void* sharedMem);
// (reference library/include/rocfft/rocfft.h:533-612).  Offsets are in elements of the array
// type (real scalars or complex pairs) from the buffer pointer given to rocfft_execute.
struct fftk_cb_params
{
    uint32_t len[3];
    uint32_t batch;
    int64_t  stride[3];
    int64_t  dist;
    int64_t  offset;
    uint32_t store; // 0: user -> scratch through the load callback, 1: scratch -> user through the store callback
    void*    user;
    void*    scratch;
    void*    fn;   // device address of the callback; null = plain copy
    void*    data; // cbdata
};

// one-workgroup 32768-point single-precision transform (big_kernels.hip)
struct fftk_big_params
{
    const void* in;
    void*       out;
    int64_t     in_line[3], out_line[3]; // strides between transforms, in scalars
    uint32_t    lines[3];
    const void* tw;     // stacked twiddles of the radix 32x32x32 schedule
    const void* half_a; // e^{-2 pi i t/65536}, t in [0, 1024)
    const void* half_b; // e^{-2 pi i k/64}, k in [0, 32)
    int32_t     dir;    // complex mode: -1 forward, +1 inverse
    uint32_t    mode;   // 0 complex, 1 real forward (65536 reals -> 32769 bins), 2 real inverse
    double      scale;
    uint32_t    use_scale;
};

#endif
