// api.cpp -- the rocfft.h entry points: handles, defaults, validation, plan
// creation and execution.  Behaviour follows the reference API glue
// (library/src/plan.cpp:69-77, :87-197, :224-285, :397-488, :729-779, :2959-3145,
// :3279-3289; library/src/transform.cpp:35-103, :331-474); the planner behind it
// is this library's own (plan.cpp).
#include "gpu_rt.h"
#include "plan.h"
#include "rocfft/rocfft.h"
#include "rocfft_amd.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

using namespace fftamd;

#define ROCFFT_AMD_VERSION "1.0.32.amd-gfx950-0.1"

struct rocfft_plan_description_t
{
    rocfft_array_type   inArrayType  = rocfft_array_type_unset;
    rocfft_array_type   outArrayType = rocfft_array_type_unset;
    std::vector<size_t> inStrides, outStrides;
    size_t              inDist = 0, outDist = 0;
    size_t              inOffset[2]  = {0, 0};
    size_t              outOffset[2] = {0, 0};
    double              scale        = 1.0;
    bool                has_scale    = false;
    bool                distributed  = false; // a field or communicator was attached
};

// Device buffers a plan keeps for executions that stage through copies (load/store callbacks,
// half precision): the copies of the input and output arrays and, when the caller sets no work
// buffer, the work area.  One set per stream the plan has been executed on.  A buffer is
// allocated by the first execution on that stream that needs it and replaced by a larger one
// when a later execution needs more; nothing is freed before the plan is destroyed (a graph
// captured earlier, or a thread that has read the pointers and not yet enqueued its kernels,
// may still use a replaced buffer), so that executions which find what they need allocate
// nothing, do not wait for the stream and can be captured into a graph.
struct StageBuf
{
    void*  ptr   = nullptr;
    size_t bytes = 0;
};
struct StageSet
{
    StageBuf in[2], out[2], work;
};

struct rocfft_plan_t
{
    Problem     prob;
    ExecPlan    exec;
    int         device = 0;
    std::string error;
    bool        half_io = false; // half-precision arrays: the plan computes in single precision on scratch copies
    // stage_lock is held from the lookup of a set until every kernel that uses its buffers has
    // been enqueued: the order of enqueueing on a stream is then the order of use
    std::mutex                stage_lock;
    std::map<void*, StageSet> stage; // by stream
    std::vector<void*>        stage_allocs; // every buffer of every set, replaced ones included
    // makes b hold at least `bytes`; false when the allocation fails
    bool stage_grow(StageBuf& b, size_t bytes)
    {
        if(b.ptr && b.bytes >= bytes)
            return true;
        void* p = nullptr;
        if(fftrt_malloc(&p, bytes) != 0)
            return false;
        stage_allocs.push_back(p);
        b.ptr   = p;
        b.bytes = bytes;
        return true;
    }
    ~rocfft_plan_t()
    {
        if(!stage_allocs.empty())
            fftrt_device_sync(); // executions in flight may still use the buffers
        for(void* p : stage_allocs)
            fftrt_free(p);
    }
};

struct rocfft_execution_info_t
{
    void*  workBuffer     = nullptr;
    size_t workBufferSize = 0;
    void*  stream         = nullptr;
    void*  load_cb        = nullptr; // device address of the load callback, its data
    void*  load_cb_data   = nullptr;
    void*  store_cb       = nullptr;
    void*  store_cb_data  = nullptr;
};

struct rocfft_field_t
{
    int bricks = 0;
};
struct rocfft_brick_t
{
    int device = 0;
};

// ---------------------------------------------------------------------------
// defaults and validation

// What a plan description may leave unset on one side (input or output) of a transform, and
// the rule of the API that completes it (the contract of the reference's defaults,
// library/src/plan.cpp:87-197; see also the in-place real layouts of rocfft.h:107-112):
//   array type  a real transform has one real and one Hermitian side, a complex one two
//               interleaved complex sides;
//   strides     packed: dimension d steps over the rows of the dimensions below it.  The real side
//               of an in-place real transform lies over the Hermitian rows, so its row 0 takes the
//               2 (n0/2 + 1) reals that row covers instead of n0;
//   distance    the extent of one transform, i.e. last length x last stride -- for rank 1 laid over
//               the Hermitian row as above.
enum SideRole
{
    SIDE_COMPLEX,
    SIDE_REAL,
    SIDE_HERMITIAN
};

static void complete_side(rocfft_array_type& type, std::vector<size_t>& stride, size_t& dist, SideRole role,
                          bool laid_over_hermitian, const std::vector<size_t>& array_len, size_t hermitian_row)
{
    if(type == rocfft_array_type_unset)
        type = role == SIDE_REAL        ? rocfft_array_type_real
               : role == SIDE_HERMITIAN ? rocfft_array_type_hermitian_interleaved
                                        : rocfft_array_type_complex_interleaved;
    const size_t rank = array_len.size();
    const size_t row0 = laid_over_hermitian ? 2 * hermitian_row : array_len[0];
    if(stride.empty())
    {
        size_t step = 1;
        for(size_t d = 0; d < rank; ++d)
        {
            stride.push_back(step);
            step *= d == 0 ? row0 : array_len[d];
        }
    }
    if(dist == 0)
        dist = (rank == 1 && laid_over_hermitian) ? row0 * stride[0] : array_len[rank - 1] * stride[rank - 1];
}

static void init_defaults(rocfft_plan_description_t& d, rocfft_transform_type type,
                          rocfft_result_placement placement, const std::vector<size_t>& in_len,
                          const std::vector<size_t>& out_len)
{
    const bool   inplace = placement == rocfft_placement_inplace;
    const bool   fwd     = type == rocfft_transform_type_real_forward;
    const bool   inv     = type == rocfft_transform_type_real_inverse;
    const size_t herm    = fwd ? out_len[0] : in_len[0]; // bins per Hermitian row (real transforms)
    complete_side(d.inArrayType, d.inStrides, d.inDist, fwd ? SIDE_REAL : inv ? SIDE_HERMITIAN : SIDE_COMPLEX,
                  fwd && inplace, in_len, herm);
    complete_side(d.outArrayType, d.outStrides, d.outDist, fwd ? SIDE_HERMITIAN : inv ? SIDE_REAL : SIDE_COMPLEX,
                  inv && inplace, out_len, herm);
}

// transform type, array types and placement must agree (reference plan.cpp:729-779)
static rocfft_status check_array_types(rocfft_transform_type type, rocfft_result_placement placement,
                                       const rocfft_plan_description_t& d)
{
    auto is_complex = [](rocfft_array_type t) {
        return t == rocfft_array_type_complex_interleaved || t == rocfft_array_type_complex_planar;
    };
    auto is_herm = [](rocfft_array_type t) {
        return t == rocfft_array_type_hermitian_interleaved || t == rocfft_array_type_hermitian_planar;
    };
    const bool inplace = placement == rocfft_placement_inplace;
    switch(type)
    {
    case rocfft_transform_type_complex_forward:
    case rocfft_transform_type_complex_inverse:
        if(!is_complex(d.inArrayType) || !is_complex(d.outArrayType))
            return rocfft_status_invalid_array_type;
        if(inplace && d.inArrayType != d.outArrayType)
            return rocfft_status_invalid_array_type;
        break;
    case rocfft_transform_type_real_forward:
        if(d.inArrayType != rocfft_array_type_real || !is_herm(d.outArrayType))
            return rocfft_status_invalid_array_type;
        if(inplace && d.outArrayType != rocfft_array_type_hermitian_interleaved)
            return rocfft_status_invalid_array_type;
        break;
    case rocfft_transform_type_real_inverse:
        if(d.outArrayType != rocfft_array_type_real || !is_herm(d.inArrayType))
            return rocfft_status_invalid_array_type;
        if(inplace && d.inArrayType != rocfft_array_type_hermitian_interleaved)
            return rocfft_status_invalid_array_type;
        break;
    default:
        return rocfft_status_invalid_arg_value;
    }
    return rocfft_status_success;
}

// Turns the API arguments into a Problem (dimension order as given; the planner
// picks its own pass order, so the reference's stride sort, plan.cpp:224-285, is
// only applied to drop unit-length trailing dimensions).
static rocfft_status make_problem(Problem& p, rocfft_result_placement placement,
                                  rocfft_transform_type type, rocfft_precision precision,
                                  size_t dimensions, const size_t* lengths, size_t batch,
                                  const rocfft_plan_description description)
{
    if(dimensions < 1 || dimensions > 3)
        return rocfft_status_invalid_dimensions;
    if(!lengths)
        return rocfft_status_failure;
    if((int)type < 0 || (int)type > 3)
        return rocfft_status_invalid_arg_value;
    std::vector<size_t> len(lengths, lengths + dimensions);
    for(size_t v : len)
        if(v == 0)
            return rocfft_status_invalid_dimensions;
    const bool is_real
        = type == rocfft_transform_type_real_forward || type == rocfft_transform_type_real_inverse;
    // array lengths on each side (reference plan.cpp:2980-2987)
    std::vector<size_t> ilen = len, olen = len;
    if(type == rocfft_transform_type_real_forward)
        olen[0] = len[0] / 2 + 1;
    if(type == rocfft_transform_type_real_inverse)
        ilen[0] = len[0] / 2 + 1;
    rocfft_plan_description_t d;
    if(description)
        d = *description;
    if(d.distributed)
        return rocfft_status_failure;
    if(!d.inStrides.empty() && d.inStrides.size() != dimensions)
        return rocfft_status_invalid_strides;
    if(!d.outStrides.empty() && d.outStrides.size() != dimensions)
        return rocfft_status_invalid_strides;
    init_defaults(d, type, placement, ilen, olen);
    rocfft_status st = check_array_types(type, placement, d);
    if(st != rocfft_status_success)
        return st;
    (void)is_real;
    memset(&p, 0, sizeof(p));
    p.type      = type;
    p.precision = precision;
    p.placement = placement;
    p.rank      = dimensions;
    p.batch     = batch;
    p.in_type   = d.inArrayType;
    p.out_type  = d.outArrayType;
    for(size_t i = 0; i < dimensions; ++i)
    {
        p.len[i]     = len[i];
        p.istride[i] = d.inStrides[i];
        p.ostride[i] = d.outStrides[i];
    }
    p.idist = d.inDist;
    p.odist = d.outDist;
    for(int i = 0; i < 2; ++i)
    {
        p.ioffset[i] = d.inOffset[i];
        p.ooffset[i] = d.outOffset[i];
    }
    p.scale     = d.scale;
    p.has_scale = d.has_scale && d.scale != 1.0;
    // trailing unit dimensions carry no work (reference plan.cpp:271-276)
    while(p.rank > 1 && p.len[p.rank - 1] == 1)
        --p.rank;
    return rocfft_status_success;
}

// ---------------------------------------------------------------------------
// entry points

static int g_setup_count = 0;

// ---------------------------------------------------------------------------
// Log layers, selected by the bits of ROCFFT_LAYER as in the reference
// (library/src/include/logging.h:139-150): 1 trace (every API call with its arguments),
// 2 bench (a rocfft-bench command line per plan, library/src/plan.cpp:698-726), 4 profile
// (duration and bandwidth of every kernel of an execute, library/src/powX.cpp:855-882),
// 8 plan (the pass list).  Each layer writes to stderr, or appends to the file named by
// ROCFFT_LOG_TRACE_PATH / _BENCH_PATH / _PROFILE_PATH / _PLAN_PATH
// (library/src/auxiliary.cpp:88-128).
enum
{
    LOG_TRACE   = 1,
    LOG_BENCH   = 2,
    LOG_PROFILE = 4,
    LOG_PLAN    = 8
};
static int        g_layers = 0;
static FILE*      g_log_file[4] = {nullptr, nullptr, nullptr, nullptr};
static std::mutex g_log_mutex;

static FILE* log_stream(int layer)
{
    int   i = layer == LOG_TRACE ? 0 : layer == LOG_BENCH ? 1 : layer == LOG_PROFILE ? 2 : 3;
    FILE* f = g_log_file[i];
    return f ? f : stderr;
}

static void log_line(int layer, const std::string& text)
{
    std::lock_guard<std::mutex> lock(g_log_mutex);
    FILE*                       f = log_stream(layer);
    fputs(text.c_str(), f);
    if(text.empty() || text.back() != '\n')
        fputc('\n', f);
    fflush(f);
}

// "function,key,value,key,value,..." as the reference's trace lines
struct TraceLine
{
    std::ostringstream o;
    bool               on;
    explicit TraceLine(const char* fn)
        : on((g_layers & LOG_TRACE) != 0)
    {
        if(on)
            o << fn;
    }
    template <typename V>
    TraceLine& arg(const char* key, const V& v)
    {
        if(on)
            o << "," << key << "," << v;
        return *this;
    }
    TraceLine& sizes(const char* key, const size_t* v, size_t n)
    {
        if(on)
        {
            o << "," << key << ",";
            for(size_t i = 0; v && i < n; ++i)
                o << (i ? " " : "") << v[i];
        }
        return *this;
    }
    ~TraceLine()
    {
        if(on)
            log_line(LOG_TRACE, o.str());
    }
};

static std::string bench_command(const Problem& p, bool half_io)
{
    std::ostringstream o;
    o << "rocfft-bench --length ";
    for(size_t d = p.rank; d-- > 0;)
        o << p.len[d] << " ";
    o << "-b " << p.batch << " ";
    if(p.placement == rocfft_placement_notinplace)
        o << "-o ";
    o << "-t " << (int)p.type << " --precision "
      << (half_io ? "half" : p.precision == rocfft_precision_double ? "double" : "single")
      << " --itype " << (int)p.in_type << " --otype " << (int)p.out_type << " --istride ";
    for(size_t d = p.rank; d-- > 0;)
        o << p.istride[d] << " ";
    o << "--ostride ";
    for(size_t d = p.rank; d-- > 0;)
        o << p.ostride[d] << " ";
    o << "--idist " << p.idist << " --odist " << p.odist << " --ioffset " << p.ioffset[0] << " "
      << p.ioffset[1] << " --ooffset " << p.ooffset[0] << " " << p.ooffset[1];
    if(p.has_scale)
        o << " --scalefactor " << p.scale;
    return o.str();
}

extern "C" {

rocfft_status rocfft_setup(void)
{
    ++g_setup_count;
    const char* layer = getenv("ROCFFT_LAYER");
    g_layers          = layer ? (int)strtol(layer, nullptr, 0) : 0;
    static const char* const path_vars[4]
        = {"ROCFFT_LOG_TRACE_PATH", "ROCFFT_LOG_BENCH_PATH", "ROCFFT_LOG_PROFILE_PATH", "ROCFFT_LOG_PLAN_PATH"};
    for(int i = 0; i < 4; ++i)
    {
        const char* path = getenv(path_vars[i]);
        if((g_layers & (1 << i)) && path && *path && !g_log_file[i])
            g_log_file[i] = fopen(path, "a");
    }
    TraceLine t(__func__);
    return rocfft_status_success;
}

rocfft_status rocfft_cleanup(void)
{
    {
        TraceLine t(__func__);
    }
    if(g_setup_count > 0)
        --g_setup_count;
    table_cache_clear();
    return rocfft_status_success;
}

rocfft_status rocfft_plan_create(rocfft_plan* plan, rocfft_result_placement placement,
                                 rocfft_transform_type transform_type, rocfft_precision precision,
                                 size_t dimensions, const size_t* lengths, size_t number_of_transforms,
                                 const rocfft_plan_description description)
{
    if(!plan)
        return rocfft_status_failure;
    *plan = nullptr;
    TraceLine(__func__)
        .arg("placement", (int)placement)
        .arg("transform_type", (int)transform_type)
        .arg("precision", (int)precision)
        .arg("dimensions", dimensions)
        .sizes("lengths", lengths, dimensions <= 3 ? dimensions : 0)
        .arg("number_of_transforms", number_of_transforms)
        .arg("description", (const void*)description);
    try
    {
        rocfft_plan_t* p = new rocfft_plan_t;
        // half precision: same layouts, single-precision arithmetic on staged copies
        p->half_io       = precision == rocfft_precision_half;
        rocfft_status st = make_problem(p->prob, placement, transform_type,
                                        p->half_io ? rocfft_precision_single : precision, dimensions, lengths,
                                        number_of_transforms, description);
        if(st == rocfft_status_success && (g_layers & LOG_BENCH))
            log_line(LOG_BENCH, bench_command(p->prob, p->half_io));
        if(st == rocfft_status_success)
        {
            int ndev = 0;
            if(fftrt_device_count(&ndev) != 0 || ndev < 1)
            {
                p->error = "no GPU available";
                st       = rocfft_status_failure;
            }
        }
        if(st == rocfft_status_success)
        {
            fftrt_device_info(&p->device, nullptr, nullptr, nullptr, 0);
            st = build_exec_plan(p->prob, p->exec, false, p->error);
        }
        if(st != rocfft_status_success)
        {
            if(getenv("ROCFFT_AMD_VERBOSE") && !p->error.empty())
                fprintf(stderr, "rocfft_plan_create: %s\n", p->error.c_str());
            delete p;
            return st;
        }
        if(g_layers & LOG_PLAN)
            log_line(LOG_PLAN, p->exec.describe());
        *plan = p;
        return rocfft_status_success;
    }
    catch(...)
    {
        return rocfft_status_failure;
    }
}

// static_work: take the work area from the library's device-resident array instead of the
// caller's buffer or a fresh allocation, and refuse whatever would need an allocation
// ROCFFT_AMD_NO_HALF_FUSE=1: half-precision arrays are always converted in separate passes
static const bool g_no_half_fuse = getenv("ROCFFT_AMD_NO_HALF_FUSE") != nullptr;

static rocfft_status execute_impl(const rocfft_plan plan, void* in_buffer[], void* out_buffer[],
                                  rocfft_execution_info info, float* pass_ms, bool static_work = false)
{
    if(!plan || !in_buffer || !in_buffer[0])
        return rocfft_status_failure;
    try
    {
        const ExecPlan& ep     = plan->exec;
        const Problem&  pr     = plan->prob;
        auto            planar = [](rocfft_array_type t) {
            return t == rocfft_array_type_complex_planar || t == rocfft_array_type_hermitian_planar;
        };
        void* in[2]  = {in_buffer[0], planar(pr.in_type) ? in_buffer[1] : nullptr};
        void* out[2] = {nullptr, nullptr};
        if(ep.inplace)
        {
            out[0] = in[0];
            out[1] = in[1];
        }
        else
        {
            if(!out_buffer || !out_buffer[0])
                return rocfft_status_failure;
            out[0] = out_buffer[0];
            out[1] = planar(pr.out_type) ? out_buffer[1] : nullptr;
        }
        if((planar(pr.in_type) && !in[1]) || (planar(pr.out_type) && !out[1]))
            return rocfft_status_failure;
        void*  stream = info ? info->stream : nullptr;
        // the work area the pass-list choice is made for: the library's static array when that
        // will be used, else the caller's buffer (null: an aligned allocation follows)
        void*  static_ptr  = nullptr;
        size_t static_have = 0;
        if(static_work && fftrt_static_scratch(&static_ptr, &static_have) != 0)
            return rocfft_status_failure;
        void* const work_hint = static_work ? static_ptr : (info ? info->workBuffer : nullptr);
        // Load/store callbacks run inside the first and last kernel when those have a callback
        // form (interleaved or real arrays); otherwise, and for half precision, the arrays are
        // staged through copies.
        const bool    have_cb = info && (info->load_cb || info->store_cb);
        const bool    half_io = plan->half_io;
        ExecCallbacks ecb;
        bool          fused = false;
        if(have_cb && !half_io && !planar(pr.in_type) && !planar(pr.out_type))
        {
            ecb.load_fn     = info->load_cb;
            ecb.load_data   = info->load_cb_data;
            ecb.store_fn    = info->store_cb;
            ecb.store_data  = info->store_cb_data;
            ecb.in_complex  = pr.in_type != rocfft_array_type_real;
            ecb.out_complex = pr.out_type != rocfft_array_type_real;
            fused           = callbacks_fusable(ep, in, out, work_hint, ecb);
        }
        const bool staging = half_io || (have_cb && !fused);
        if(staging && have_cb && (planar(pr.in_type) || planar(pr.out_type) || half_io))
            return rocfft_status_failure;
        // the work area of the pass list these buffers get (staged copies are aligned allocations)
        size_t need = staging ? ep.work_bytes()
                              : select_exec_plan(ep, in, out, work_hint, fused ? &ecb : nullptr).own_work_bytes();
        void* work = nullptr;
        bool  own  = false;
        if(need && static_work)
        {
            if(need > static_have)
            {
                fprintf(stderr,
                        "rocfft_amd_execute_static: the plan needs %zu bytes of work area, the static area "
                        "holds %zu\n",
                        need, static_have);
                return rocfft_status_invalid_work_buffer;
            }
            work = static_ptr;
        }
        else if(need)
        {
            if(info && info->workBuffer)
            {
                if(info->workBufferSize < need)
                    return rocfft_status_invalid_work_buffer;
                work = info->workBuffer;
            }
            else if(!staging)
            {
                // no caller-owned scratch: allocate for this call (reference
                // transform.cpp:424-434); impossible while the stream is being captured
                if(fftrt_stream_capturing(stream))
                    return rocfft_status_invalid_work_buffer;
                if(fftrt_malloc(&work, need) != 0)
                    return rocfft_status_failure;
                own = true;
            }
        }
        if(pass_ms && fftrt_stream_capturing(stream))
            return rocfft_status_failure;
        auto cleanup = [&]() {
            if(own)
            {
                fftrt_stream_sync(stream);
                fftrt_free(work);
            }
        };

        // Staging.  Load/store callbacks no kernel of the pass list can call: the input is copied
        // into a scratch buffer of the same layout through the load callback, the plan runs on
        // scratch buffers, and the result goes to the user's buffer through the store callback.
        // Half precision: the plan computes in single precision; a first (last) pass that converts
        // on load (store) takes the user's half array itself, every other access to the input
        // (output) array goes to a single-precision scratch array of the same layout, which a
        // copy fills from (writes back to) the user's array when the pass on that side cannot
        // convert.  The scratch arrays belong to the plan (one set per stream, see StageSet).
        void*          st_in[2]  = {nullptr, nullptr};
        void*          st_out[2] = {nullptr, nullptr};
        fftk_cb_params cin, cout;
        memset(&cin, 0, sizeof(cin));
        memset(&cout, 0, sizeof(cout));
        const bool in_planar = planar(pr.in_type), out_planar = planar(pr.out_type);
        // elements of one buffer are complex pairs only for interleaved complex arrays
        const bool in_complex  = pr.in_type != rocfft_array_type_real && !in_planar;
        const bool out_complex = pr.out_type != rocfft_array_type_real && !out_planar;
        const int  nin = in_planar ? 2 : 1, nout = out_planar ? 2 : 1;
        bool       stage_in = false, stage_out = false; // that side has a scratch array
        bool       copy_in = false, copy_out = false;   // ... which a separate pass fills / writes back
        ExecHalf   ehalf;
        std::unique_lock<std::mutex> stage_guard(plan->stage_lock, std::defer_lock);
        if(staging)
        {
            const size_t scalar = ep.precision ? 8 : 4; // of the scratch arrays
            auto         fill   = [&](fftk_cb_params& c, bool input) {
                size_t off0   = input ? std::max(pr.ioffset[0], pr.ioffset[1]) : std::max(pr.ooffset[0], pr.ooffset[1]);
                size_t extent = off0 + 1;
                for(size_t d = 0; d < 3; ++d)
                {
                    size_t n = d < pr.rank ? pr.len[d] : 1;
                    if(d == 0 && ((input && pr.type == rocfft_transform_type_real_inverse)
                                  || (!input && pr.type == rocfft_transform_type_real_forward)))
                        n = n / 2 + 1;
                    c.len[d]    = (uint32_t)n;
                    c.stride[d] = d < pr.rank ? (int64_t)(input ? pr.istride[d] : pr.ostride[d]) : 0;
                    extent += (n - 1) * (size_t)c.stride[d];
                }
                c.batch = (uint32_t)pr.batch;
                c.dist  = (int64_t)(input ? pr.idist : pr.odist);
                extent += (pr.batch - 1) * (size_t)c.dist;
                return extent * scalar * ((input ? in_complex : out_complex) ? 2 : 1);
            };
            size_t       in_bytes  = fill(cin, true);
            const size_t out_bytes = fill(cout, false);
            if(ep.inplace)
                in_bytes = std::max(in_bytes, out_bytes);
            stage_in  = ep.inplace || half_io || info->load_cb;
            stage_out = ep.inplace || half_io || info->store_cb;
            copy_in   = stage_in;
            copy_out  = stage_out;
            // half precision: which sides the kernels convert themselves, and which scratch arrays
            // the pass list then still touches.  (The scratch arrays and an allocated work area are
            // aligned allocations: only a caller's work buffer can send the choice to the other
            // pass list, which has no converting kernels.)
            if(half_io && !g_no_half_fuse)
            {
                void* const aligned_stub   = reinterpret_cast<void*>(uintptr_t(4096));
                void*       probe[2]       = {aligned_stub, aligned_stub};
                const void* const probe_wk = work ? work : aligned_stub;
                if(&select_exec_plan(ep, probe, probe, probe_wk) == &ep)
                {
                    ehalf.in       = in[0];
                    ehalf.out      = out[0];
                    ehalf.fuse_in  = !in_planar && half_fusable(ep, true, in[0]);
                    ehalf.fuse_out = !out_planar && half_fusable(ep, false, out[0]);
                    half_scratch_needs(ep, ehalf.fuse_in, ehalf.fuse_out, stage_in, stage_out);
                    copy_in  = !ehalf.fuse_in;
                    copy_out = !ehalf.fuse_out;
                    if(ep.inplace)
                        stage_in = stage_out = stage_in || stage_out;
                }
            }
            const size_t want_work = (need && !work) ? need : 0;
            if(stage_in || stage_out || want_work)
            {
                stage_guard.lock();
                StageSet&  set  = plan->stage[stream];
                const bool fits = (!stage_in || (set.in[0].bytes >= in_bytes && (nin < 2 || set.in[1].bytes >= in_bytes)))
                                  && (!stage_out || ep.inplace
                                      || (set.out[0].bytes >= out_bytes && (nout < 2 || set.out[1].bytes >= out_bytes)))
                                  && set.work.bytes >= want_work;
                if(!fits)
                {
                    // allocating: not in the variant that may not, and not while the stream is
                    // being captured
                    if(static_work || fftrt_stream_capturing(stream))
                        return rocfft_status_failure;
                    bool ok = true;
                    for(int i = 0; i < nin && ok && stage_in; ++i)
                        ok = plan->stage_grow(set.in[i], in_bytes);
                    for(int i = 0; i < nout && ok && stage_out && !ep.inplace; ++i)
                        ok = plan->stage_grow(set.out[i], out_bytes);
                    if(ok && want_work)
                        ok = plan->stage_grow(set.work, want_work);
                    if(!ok)
                        return rocfft_status_failure;
                }
                for(int i = 0; i < 2; ++i)
                {
                    st_in[i]  = stage_in ? set.in[i].ptr : nullptr;
                    st_out[i] = stage_out ? (ep.inplace ? set.in[i].ptr : set.out[i].ptr) : nullptr;
                }
                if(want_work)
                    work = set.work.ptr;
            }
            bool ok = true;
            for(int i = 0; i < nin && ok && copy_in; ++i)
            {
                cin.store   = 0;
                cin.offset  = (int64_t)pr.ioffset[i];
                cin.user    = in[i];
                cin.scratch = st_in[i];
                cin.fn      = half_io ? nullptr : info->load_cb;
                cin.data    = half_io ? nullptr : info->load_cb_data;
                ok = (half_io ? fftrt_launch_half_copy(&cin, in_complex ? 1 : 0, stream)
                              : fftrt_launch_callback_copy(&cin, ep.precision, in_complex ? 1 : 0, stream))
                     == 0;
            }
            if(!ok)
                return rocfft_status_failure;
        }
        // (a side without scratch array that the kernels convert themselves: the pointer handed on
        // is never used, the pass takes ehalf.in / ehalf.out)
        void* run_in[2]  = {stage_in ? st_in[0] : in[0], stage_in ? st_in[1] : in[1]};
        void* run_out[2] = {stage_out ? st_out[0] : out[0], stage_out ? st_out[1] : out[1]};
        rocfft_status st = run_exec_plan(ep, run_in, run_out, work, stream, pass_ms, fused ? &ecb : nullptr,
                                         (ehalf.fuse_in || ehalf.fuse_out) ? &ehalf : nullptr);
        for(int i = 0; i < nout && st == rocfft_status_success && copy_out; ++i)
        {
            cout.store   = 1;
            cout.offset  = (int64_t)pr.ooffset[i];
            cout.user    = out[i];
            cout.scratch = st_out[i];
            cout.fn      = half_io ? nullptr : info->store_cb;
            cout.data    = half_io ? nullptr : info->store_cb_data;
            int rc       = half_io ? fftrt_launch_half_copy(&cout, out_complex ? 1 : 0, stream)
                                   : fftrt_launch_callback_copy(&cout, ep.precision, out_complex ? 1 : 0, stream);
            if(rc != 0)
                st = rocfft_status_failure;
        }
        cleanup();
        return st;
    }
    catch(...)
    {
        return rocfft_status_failure;
    }
}

rocfft_status rocfft_execute(const rocfft_plan plan, void* in_buffer[], void* out_buffer[],
                             rocfft_execution_info info)
{
    TraceLine(__func__)
        .arg("plan", (const void*)plan)
        .arg("in_buffer", in_buffer ? in_buffer[0] : nullptr)
        .arg("out_buffer", out_buffer ? out_buffer[0] : nullptr)
        .arg("info", (const void*)info);
    // the profile layer times every kernel with events and waits for them, as the reference's
    // does; it is skipped while the stream is being captured
    if((g_layers & LOG_PROFILE) && plan && !fftrt_stream_capturing(info ? info->stream : nullptr))
    {
        std::vector<float> ms(plan->exec.passes.size() + 1, 0.0f);
        rocfft_status      st = execute_impl(plan, in_buffer, out_buffer, info, ms.data());
        if(st != rocfft_status_success)
            return st;
        const double peak = 8000.0; // GB/s, HBM3E of MI355X
        for(size_t i = 0; i < plan->exec.passes.size(); ++i)
        {
            const PassRec&     r  = plan->exec.passes[i];
            const double       bw = ms[i] > 0 ? r.bytes_rw / (ms[i] * 1e6) : 0.0;
            std::ostringstream o;
            o << "TransformPowX,scheme," << r.note << ",duration_ms," << ms[i] << ",total_size_bytes,"
              << (uint64_t)r.bytes_rw << ",exec_GB_s," << bw << ",max_mem_GB_s," << peak
              << ",bw_efficiency_pct," << 100.0 * bw / peak << ",kernel_index," << i;
            log_line(LOG_PROFILE, o.str());
        }
        return st;
    }
    return execute_impl(plan, in_buffer, out_buffer, info, nullptr);
}

rocfft_status rocfft_amd_execute_profile(const rocfft_plan plan, void* in_buffer[], void* out_buffer[],
                                         rocfft_execution_info info, float* pass_ms, size_t capacity)
{
    if(!plan || !pass_ms || capacity < plan->exec.passes.size())
        return rocfft_status_invalid_arg_value;
    return execute_impl(plan, in_buffer, out_buffer, info, pass_ms);
}

rocfft_status rocfft_amd_execute_static(const rocfft_plan plan, void* in_buffer[], void* out_buffer[],
                                        rocfft_execution_info info)
{
    return execute_impl(plan, in_buffer, out_buffer, info, nullptr, true);
}

rocfft_status rocfft_amd_copy_probe(const rocfft_amd_probe* probe, void* stream)
{
    if(!probe)
        return rocfft_status_invalid_arg_value;
    return fftrt_copy_probe(probe, stream) == 0 ? rocfft_status_success : rocfft_status_failure;
}

rocfft_status rocfft_amd_plan_get_pass_count(const rocfft_plan plan, size_t* count)
{
    if(!plan || !count)
        return rocfft_status_failure;
    *count = plan->exec.passes.size();
    return rocfft_status_success;
}

rocfft_status rocfft_amd_plan_get_pass_info(const rocfft_plan plan, size_t index, char* name,
                                            size_t name_len, double* bytes_read_written)
{
    if(!plan || index >= plan->exec.passes.size())
        return rocfft_status_invalid_arg_value;
    const PassRec& r = plan->exec.passes[index];
    if(name && name_len)
    {
        size_t ncopy = std::min(name_len - 1, r.note.size());
        memcpy(name, r.note.data(), ncopy);
        name[ncopy] = 0;
    }
    if(bytes_read_written)
        *bytes_read_written = r.bytes_rw;
    return rocfft_status_success;
}

rocfft_status rocfft_plan_destroy(rocfft_plan plan)
{
    TraceLine(__func__).arg("plan", (const void*)plan);
    delete plan;
    return rocfft_status_success;
}

rocfft_status rocfft_plan_description_set_scale_factor(rocfft_plan_description description,
                                                       const double            scale_factor)
{
    TraceLine(__func__).arg("description", (const void*)description).arg("scale", scale_factor);
    if(!description)
        return rocfft_status_failure;
    if(!std::isfinite(scale_factor))
        return rocfft_status_invalid_arg_value;
    description->scale     = scale_factor;
    description->has_scale = true;
    return rocfft_status_success;
}

rocfft_status rocfft_plan_description_set_data_layout(rocfft_plan_description description,
                                                      const rocfft_array_type in_array_type,
                                                      const rocfft_array_type out_array_type,
                                                      const size_t*           in_offsets,
                                                      const size_t*           out_offsets,
                                                      const size_t            in_strides_size,
                                                      const size_t*           in_strides,
                                                      const size_t            in_distance,
                                                      const size_t            out_strides_size,
                                                      const size_t*           out_strides,
                                                      const size_t            out_distance)
{
    TraceLine(__func__)
        .arg("description", (const void*)description)
        .arg("in_array_type", (int)in_array_type)
        .arg("out_array_type", (int)out_array_type)
        .sizes("in_offsets", in_offsets, 2)
        .sizes("out_offsets", out_offsets, 2)
        .sizes("in_strides", in_strides, in_strides_size <= 3 ? in_strides_size : 0)
        .arg("in_distance", in_distance)
        .sizes("out_strides", out_strides, out_strides_size <= 3 ? out_strides_size : 0)
        .arg("out_distance", out_distance);
    if(!description)
        return rocfft_status_failure;
    auto planar = [](rocfft_array_type t) {
        return t == rocfft_array_type_complex_planar || t == rocfft_array_type_hermitian_planar;
    };
    description->inArrayType  = in_array_type;
    description->outArrayType = out_array_type;
    if(in_offsets)
    {
        description->inOffset[0] = in_offsets[0];
        if(planar(in_array_type))
            description->inOffset[1] = in_offsets[1];
    }
    if(out_offsets)
    {
        description->outOffset[0] = out_offsets[0];
        if(planar(out_array_type))
            description->outOffset[1] = out_offsets[1];
    }
    if(in_strides)
        description->inStrides.assign(in_strides, in_strides + in_strides_size);
    if(in_distance)
        description->inDist = in_distance;
    if(out_strides)
        description->outStrides.assign(out_strides, out_strides + out_strides_size);
    if(out_distance)
        description->outDist = out_distance;
    return rocfft_status_success;
}

rocfft_status rocfft_field_create(rocfft_field* field)
{
    if(!field)
        return rocfft_status_failure;
    *field = new rocfft_field_t;
    return rocfft_status_success;
}
rocfft_status rocfft_field_destroy(rocfft_field field)
{
    delete field;
    return rocfft_status_success;
}

rocfft_status rocfft_get_version_string(char* buf, size_t len)
{
    static const char v[] = ROCFFT_AMD_VERSION;
    if(!buf)
        return rocfft_status_failure;
    if(len < sizeof(v))
        return rocfft_status_invalid_arg_value;
    memcpy(buf, v, sizeof(v));
    return rocfft_status_success;
}

rocfft_status rocfft_plan_description_set_comm(rocfft_plan_description description,
                                               rocfft_comm_type comm_type, void* comm_handle)
{
    (void)comm_handle;
    if(!description)
        return rocfft_status_failure;
    if(comm_type != rocfft_comm_none)
        description->distributed = true;
    return rocfft_status_success;
}

rocfft_status rocfft_brick_create(rocfft_brick* brick, const size_t* field_lower,
                                  const size_t* field_upper, const size_t* brick_stride, size_t dim,
                                  int deviceID)
{
    if(!brick || !field_lower || !field_upper || !brick_stride || dim == 0)
        return rocfft_status_failure;
    *brick           = new rocfft_brick_t;
    (*brick)->device = deviceID;
    return rocfft_status_success;
}
rocfft_status rocfft_brick_destroy(rocfft_brick brick)
{
    delete brick;
    return rocfft_status_success;
}
rocfft_status rocfft_field_add_brick(rocfft_field field, rocfft_brick brick)
{
    if(!field || !brick)
        return rocfft_status_failure;
    ++field->bricks;
    return rocfft_status_success;
}
rocfft_status rocfft_plan_description_add_infield(rocfft_plan_description description,
                                                  rocfft_field            field)
{
    if(!description || !field)
        return rocfft_status_failure;
    description->distributed = true;
    return rocfft_status_success;
}
rocfft_status rocfft_plan_description_add_outfield(rocfft_plan_description description,
                                                   rocfft_field            field)
{
    if(!description || !field)
        return rocfft_status_failure;
    description->distributed = true;
    return rocfft_status_success;
}

rocfft_status rocfft_plan_get_work_buffer_size(const rocfft_plan plan, size_t* size_in_bytes)
{
    TraceLine(__func__).arg("plan", (const void*)plan);
    if(!plan || !size_in_bytes)
        return rocfft_status_failure;
    *size_in_bytes = plan->exec.work_bytes();
    return rocfft_status_success;
}

rocfft_status rocfft_plan_get_print(const rocfft_plan plan)
{
    if(!plan)
        return rocfft_status_failure;
    fputs(plan->exec.describe().c_str(), stdout);
    fflush(stdout);
    return rocfft_status_success;
}

rocfft_status rocfft_plan_description_create(rocfft_plan_description* description)
{
    TraceLine(__func__).arg("description", (const void*)description);
    if(!description)
        return rocfft_status_failure;
    *description = new rocfft_plan_description_t;
    return rocfft_status_success;
}
rocfft_status rocfft_plan_description_destroy(rocfft_plan_description description)
{
    TraceLine(__func__).arg("description", (const void*)description);
    delete description;
    return rocfft_status_success;
}

rocfft_status rocfft_execution_info_create(rocfft_execution_info* info)
{
    TraceLine(__func__).arg("info", (const void*)info);
    if(!info)
        return rocfft_status_failure;
    *info = new rocfft_execution_info_t;
    return rocfft_status_success;
}
rocfft_status rocfft_execution_info_destroy(rocfft_execution_info info)
{
    TraceLine(__func__).arg("info", (const void*)info);
    delete info;
    return rocfft_status_success;
}

rocfft_status rocfft_execution_info_set_work_buffer(rocfft_execution_info info, void* work_buffer,
                                                    const size_t size_in_bytes)
{
    TraceLine(__func__).arg("info", (const void*)info).arg("work_buffer", (const void*)work_buffer).arg("size_in_bytes", size_in_bytes);
    if(!info)
        return rocfft_status_failure;
    if(!work_buffer)
        return rocfft_status_invalid_work_buffer;
    info->workBuffer     = work_buffer;
    info->workBufferSize = size_in_bytes;
    return rocfft_status_success;
}

rocfft_status rocfft_execution_info_set_stream(rocfft_execution_info info, void* stream)
{
    TraceLine(__func__).arg("info", (const void*)info).arg("stream", (const void*)stream);
    if(!info)
        return rocfft_status_failure;
    info->stream = stream;
    return rocfft_status_success;
}

rocfft_status rocfft_execution_info_set_load_callback(rocfft_execution_info info, void** cb_functions,
                                                      void** cb_data, size_t shared_mem_bytes)
{
    if(!info)
        return rocfft_status_failure;
    if(shared_mem_bytes)
        return rocfft_status_invalid_arg_value;
    info->load_cb      = cb_functions ? cb_functions[0] : nullptr;
    info->load_cb_data = (info->load_cb && cb_data) ? cb_data[0] : nullptr;
    return rocfft_status_success;
}
rocfft_status rocfft_execution_info_set_store_callback(rocfft_execution_info info, void** cb_functions,
                                                       void** cb_data, size_t shared_mem_bytes)
{
    if(!info)
        return rocfft_status_failure;
    if(shared_mem_bytes)
        return rocfft_status_invalid_arg_value;
    info->store_cb      = cb_functions ? cb_functions[0] : nullptr;
    info->store_cb_data = (info->store_cb && cb_data) ? cb_data[0] : nullptr;
    return rocfft_status_success;
}

rocfft_status rocfft_cache_serialize(void** buffer, size_t* buffer_len_bytes)
{
    if(!buffer || !buffer_len_bytes)
        return rocfft_status_failure;
    *buffer           = malloc(1);
    *buffer_len_bytes = 0;
    return rocfft_status_success;
}
rocfft_status rocfft_cache_buffer_free(void* buffer)
{
    free(buffer);
    return rocfft_status_success;
}
rocfft_status rocfft_cache_deserialize(const void* buffer, size_t buffer_len_bytes)
{
    (void)buffer_len_bytes;
    if(!buffer)
        return rocfft_status_failure;
    return rocfft_status_success;
}

// ---------------------------------------------------------------------------
// extension: plan description without touching a device

rocfft_status rocfft_amd_plan_describe(rocfft_result_placement placement,
                                       rocfft_transform_type transform_type, rocfft_precision precision,
                                       size_t dimensions, const size_t* lengths,
                                       size_t number_of_transforms,
                                       const rocfft_plan_description description, char* text,
                                       size_t text_len, size_t* work_buffer_bytes)
{
    try
    {
        Problem       prob;
        // (half precision plans compute in single precision on staged copies)
        rocfft_status st = make_problem(prob, placement, transform_type,
                                        precision == rocfft_precision_half ? rocfft_precision_single : precision,
                                        dimensions, lengths,
                                        number_of_transforms, description);
        if(st != rocfft_status_success)
            return st;
        ExecPlan    ep;
        std::string err;
        st = build_exec_plan(prob, ep, true, err);
        std::string out = st == rocfft_status_success ? ep.describe() : ("error: " + err + "\n");
        if(text && text_len)
        {
            size_t ncopy = std::min(text_len - 1, out.size());
            memcpy(text, out.data(), ncopy);
            text[ncopy] = 0;
        }
        if(work_buffer_bytes)
            *work_buffer_bytes = st == rocfft_status_success ? ep.work_bytes() : 0;
        return st;
    }
    catch(...)
    {
        return rocfft_status_failure;
    }
}
}
