// plan.h -- host-side plan model: a transform becomes a short list of passes,
// each one launch of a precompiled kernel.  Plain C++, no HIP types; the GPU is
// reached only through gpu_rt.h.
//
// Reference counterparts: the tree of TreeNode/LeafNode objects and ExecPlan
// (library/src/include/tree_node.h:254-673, :1220-1323) built by
// NodeFactory (library/src/node_factory.cpp:474-834) and executed by
// TransformPowX (library/src/powX.cpp:525-957).  This planner emits the leaf
// sequence directly instead of building and then fusing a tree.
#ifndef ROCFFT_AMD_PLAN_H
#define ROCFFT_AMD_PLAN_H

#include "kparams.h"
#include "rocfft/rocfft.h"
#include <algorithm>
#include <memory>
#include <string>
#include <vector>

namespace fftamd
{

enum BufId
{
    BUF_IN  = 0, // user input
    BUF_OUT = 1, // user output
    BUF_TMP = 2, // work buffer, general scratch region
    BUF_BLU = 3, // work buffer, Bluestein region
    BUF_CPX = 4  // work buffer, complex copy of a real transform's rows
};

// a device-resident table, shared between plans through the table cache
struct DeviceTable
{
    void*  dptr  = nullptr;
    size_t bytes = 0;
    ~DeviceTable();
};
typedef std::shared_ptr<DeviceTable> TablePtr;

// the transform as the API describes it, after defaults have been filled in
struct Problem
{
    rocfft_transform_type   type;
    rocfft_precision        precision;
    rocfft_result_placement placement;
    size_t                  rank;
    size_t                  len[3]; // transform lengths (real lengths for real transforms)
    size_t                  batch;
    rocfft_array_type       in_type, out_type;
    size_t                  istride[3], ostride[3], idist, odist;
    size_t                  ioffset[2], ooffset[2];
    double                  scale;
    bool                    has_scale;
};

enum PassKind
{
    PASS_TILE      = 0,
    PASS_REAL_POST = 1,
    PASS_REAL_PRE  = 2,
    PASS_BIG       = 3, // one-workgroup 32768-point single-precision kernel
    PASS_COPY      = 4, // element-wise row copy between array kinds
    PASS_2D        = 5  // one-workgroup small 2D complex transform (kp holds its parameters)
};

// where a pass finds one side of its data: buffer, planar or not, scalar offsets
struct IoRef
{
    int     buf      = BUF_IN;
    bool    planar   = false;
    int64_t im_delta = 1; // scalars from a real part to its imaginary part (non planar)
    int64_t off0     = 0; // scalar offset of the first element (real-part array)
    int64_t off1     = 0; // scalar offset in the imaginary-part array (planar)
};

struct PassRec
{
    PassKind              kind = PASS_TILE;
    fftk_params           kp;
    fftk_real_params      rp;
    fftk_big_params       bp;
    fftk_copy_params      cp;
    IoRef                 src, dst;
    bool                  vec_ok = false;
    bool                  lean_ok = false; // eligible for the branch-free addressing path when vec holds
    uint32_t              grid   = 0;
    size_t                lds    = 0;
    std::string           note;
    double                bytes_rw = 0; // data bytes the pass reads plus writes (tables excluded)
    std::vector<TablePtr> tables; // keeps the device tables alive
};

struct ExecPlan
{
    std::vector<PassRec> passes;
    int                  precision  = 0; // 0 float, 1 double
    size_t               tmp_elems  = 0; // complex elements of general scratch
    size_t               blu_elems  = 0; // complex elements of Bluestein scratch
    size_t               cpx_elems  = 0; // complex elements of the real-as-complex scratch
    size_t               elem_bytes = 8; // bytes per complex element
    bool                 inplace    = false;
    // Passes whose kernels move (re, im) pairs with one access and have no scalar-access form
    // (the one-workgroup 32768-point and small-2D kernels, compiled kernels with more than 512
    // threads) cannot take buffers that are only aligned to a scalar.  A plan with such passes
    // carries a second pass list made of run-time-schedule tile passes only, used by the
    // executor when a buffer fails the alignment test (the reference accepts such buffers).
    std::shared_ptr<ExecPlan> unaligned;
    size_t                    own_work_bytes() const
    {
        return (tmp_elems + blu_elems + cpx_elems) * elem_bytes;
    }
    size_t work_bytes() const
    {
        return unaligned ? std::max(own_work_bytes(), unaligned->own_work_bytes()) : own_work_bytes();
    }
    std::string describe() const;
};

// Builds the pass list.  With dry_run no device memory is touched (tables get
// null device pointers), so the planner can be exercised without a GPU.
rocfft_status build_exec_plan(const Problem& prob, ExecPlan& plan, bool dry_run, std::string& err);

// Load/store callbacks of one execution (device function pointers with the reference's
// signatures, library/include/rocfft/rocfft.h:533-612).  They are called from inside the first
// and the last kernel of the pass list; those two run as the run-time-schedule kernels, which
// have the callback form of every load and store.
struct ExecCallbacks
{
    void* load_fn     = nullptr;
    void* load_data   = nullptr;
    void* store_fn    = nullptr;
    void* store_data  = nullptr;
    bool  in_complex  = false; // the callback's element is a complex pair (interleaved arrays)
    bool  out_complex = false;
};

// Half-precision plans compute in single precision.  Where the first (last) pass of the list is
// a compiled kernel that converts on load (store), it reads (writes) the user's half array
// itself; the other passes, and the sides that cannot, work on single-precision scratch arrays.
struct ExecHalf
{
    void* in       = nullptr; // the user's input array of half values (interleaved or real)
    void* out      = nullptr;
    bool  fuse_in  = false;
    bool  fuse_out = false;
};
// can the first (input = true) / last pass of the list take the user's half array at `user`?
bool half_fusable(const ExecPlan& plan, bool input, const void* user);
// Which single-precision scratch arrays (standing in for the user's input and output arrays) the
// pass list still touches when its first pass reads (fuse_in) / its last pass writes (fuse_out)
// the user's half array itself.  In place there is one array: both answers are the same.
void half_scratch_needs(const ExecPlan& plan, bool fuse_in, bool fuse_out, bool& need_in, bool& need_out);

// Enqueues every pass on `stream`.  in/out hold one pointer (interleaved, real)
// or two (planar).  `work` must hold plan.work_bytes() bytes when that is non-zero.
// When pass_ms is not null every pass is bracketed by events and its duration in
// milliseconds is written there (the call then waits for the stream).
rocfft_status run_exec_plan(const ExecPlan& plan, void* const in[2], void* const out[2], void* work,
                            void* stream, float* pass_ms = nullptr, const ExecCallbacks* cb = nullptr,
                            const ExecHalf* half = nullptr);

// The pass list run_exec_plan will use for these buffers: the plan itself, or its `unaligned`
// list when a buffer fails the alignment one of the plan's passes needs.  `work` may be null
// (not allocated yet: allocations are aligned).
const ExecPlan& select_exec_plan(const ExecPlan& plan, void* const in[2], void* const out[2], const void* work,
                                 const ExecCallbacks* cb = nullptr);

// Can the pass list these buffers get call the callbacks from inside its first and last kernel?
// (If not, the caller stages the arrays through copies instead.)
bool callbacks_fusable(const ExecPlan& plan, void* const in[2], void* const out[2], const void* work,
                       const ExecCallbacks& cb);

// drops cached tables that no plan uses any more
void table_cache_clear();

} // namespace fftamd

#endif
