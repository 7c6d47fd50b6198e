"""ctypes mirror of include/rocfft/rocfft.h (same names, argument meaning and
status codes as the reference interface, library/include/rocfft/rocfft.h).

Buffers are raw device addresses (ints); callers own all device memory, e.g.
``torch.Tensor.data_ptr()``.  Nothing here computes: every method is one call
into the shared library.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))

# enum values of rocfft.h
(STATUS_SUCCESS, STATUS_FAILURE, STATUS_INVALID_ARG_VALUE, STATUS_INVALID_DIMENSIONS,
 STATUS_INVALID_ARRAY_TYPE, STATUS_INVALID_STRIDES, STATUS_INVALID_DISTANCE,
 STATUS_INVALID_OFFSET, STATUS_INVALID_WORK_BUFFER) = range(9)
STATUS = {
    0: "rocfft_status_success",
    1: "rocfft_status_failure",
    2: "rocfft_status_invalid_arg_value",
    3: "rocfft_status_invalid_dimensions",
    4: "rocfft_status_invalid_array_type",
    5: "rocfft_status_invalid_strides",
    6: "rocfft_status_invalid_distance",
    7: "rocfft_status_invalid_offset",
    8: "rocfft_status_invalid_work_buffer",
}
COMPLEX_FORWARD, COMPLEX_INVERSE, REAL_FORWARD, REAL_INVERSE = range(4)
SINGLE, DOUBLE, HALF = range(3)
INPLACE, NOTINPLACE = range(2)
(COMPLEX_INTERLEAVED, COMPLEX_PLANAR, REAL, HERMITIAN_INTERLEAVED, HERMITIAN_PLANAR,
 UNSET) = range(6)


class RocfftError(RuntimeError):
    def __init__(self, status, what):
        super().__init__("%s returned %s" % (what, STATUS.get(status, status)))
        self.status = status


def library_path():
    """the product library; ROCFFT_AMD_LIBRARY names another build of it (experiments)"""
    return os.environ.get("ROCFFT_AMD_LIBRARY") or os.path.join(_HERE, "lib", "librocfft_amd.so")


_c_size_p = ctypes.POINTER(ctypes.c_size_t)
_c_void_pp = ctypes.POINTER(ctypes.c_void_p)

_PROTOTYPES = {
    "rocfft_setup": [],
    "rocfft_cleanup": [],
    "rocfft_plan_create": [_c_void_pp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_size_t,
                           _c_size_p, ctypes.c_size_t, ctypes.c_void_p],
    "rocfft_execute": [ctypes.c_void_p, _c_void_pp, _c_void_pp, ctypes.c_void_p],
    "rocfft_plan_destroy": [ctypes.c_void_p],
    "rocfft_plan_description_set_scale_factor": [ctypes.c_void_p, ctypes.c_double],
    "rocfft_plan_description_set_data_layout": [ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                                _c_size_p, _c_size_p, ctypes.c_size_t, _c_size_p,
                                                ctypes.c_size_t, ctypes.c_size_t, _c_size_p,
                                                ctypes.c_size_t],
    "rocfft_field_create": [_c_void_pp],
    "rocfft_field_destroy": [ctypes.c_void_p],
    "rocfft_get_version_string": [ctypes.c_char_p, ctypes.c_size_t],
    "rocfft_plan_description_set_comm": [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    "rocfft_brick_create": [_c_void_pp, _c_size_p, _c_size_p, _c_size_p, ctypes.c_size_t,
                            ctypes.c_int],
    "rocfft_brick_destroy": [ctypes.c_void_p],
    "rocfft_field_add_brick": [ctypes.c_void_p, ctypes.c_void_p],
    "rocfft_plan_description_add_infield": [ctypes.c_void_p, ctypes.c_void_p],
    "rocfft_plan_description_add_outfield": [ctypes.c_void_p, ctypes.c_void_p],
    "rocfft_plan_get_work_buffer_size": [ctypes.c_void_p, _c_size_p],
    "rocfft_plan_get_print": [ctypes.c_void_p],
    "rocfft_plan_description_create": [_c_void_pp],
    "rocfft_plan_description_destroy": [ctypes.c_void_p],
    "rocfft_execution_info_create": [_c_void_pp],
    "rocfft_execution_info_destroy": [ctypes.c_void_p],
    "rocfft_execution_info_set_work_buffer": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t],
    "rocfft_execution_info_set_stream": [ctypes.c_void_p, ctypes.c_void_p],
    "rocfft_execution_info_set_load_callback": [ctypes.c_void_p, _c_void_pp, _c_void_pp,
                                                ctypes.c_size_t],
    "rocfft_execution_info_set_store_callback": [ctypes.c_void_p, _c_void_pp, _c_void_pp,
                                                 ctypes.c_size_t],
    "rocfft_cache_serialize": [_c_void_pp, _c_size_p],
    "rocfft_cache_buffer_free": [ctypes.c_void_p],
    "rocfft_cache_deserialize": [ctypes.c_void_p, ctypes.c_size_t],
    "rocfft_amd_plan_describe": [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_size_t, _c_size_p,
                                 ctypes.c_size_t, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t,
                                 _c_size_p],
    "rocfft_amd_plan_get_pass_count": [ctypes.c_void_p, _c_size_p],
    "rocfft_amd_plan_get_pass_info": [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_char_p, ctypes.c_size_t,
                                      ctypes.POINTER(ctypes.c_double)],
    "rocfft_amd_execute_profile": [ctypes.c_void_p, _c_void_pp, _c_void_pp, ctypes.c_void_p,
                                   ctypes.POINTER(ctypes.c_float), ctypes.c_size_t],
    "rocfft_amd_execute_static": [ctypes.c_void_p, _c_void_pp, _c_void_pp, ctypes.c_void_p],
    "rocfft_amd_copy_probe": [ctypes.c_void_p, ctypes.c_void_p],
}


class Probe(ctypes.Structure):
    """rocfft_amd_probe of include/rocfft_amd.h: one plain copy in the access shape of a pass"""
    _fields_ = [("shape", ctypes.c_int), ("src", ctypes.c_void_p), ("dst", ctypes.c_void_p),
                ("bytes", ctypes.c_size_t), ("nontemporal", ctypes.c_int), ("workgroups_per_cu", ctypes.c_uint),
                ("group", ctypes.c_uint), ("rows", ctypes.c_uint), ("in_row", ctypes.c_size_t),
                ("out_row", ctypes.c_size_t), ("tile_width", ctypes.c_uint), ("elem_bytes", ctypes.c_uint),
                ("tiles_per_slab", ctypes.c_uint), ("in_slab", ctypes.c_size_t), ("out_slab", ctypes.c_size_t),
                ("resident_grid", ctypes.c_int), ("xcd_ranges", ctypes.c_int),
                ("slabs_inner", ctypes.c_uint), ("in_slab_outer", ctypes.c_size_t), ("out_slab_outer", ctypes.c_size_t)]


PROBE_STREAM, PROBE_READ, PROBE_WRITE, PROBE_ROWS, PROBE_TILES = range(5)

# size of the device-resident work area behind rocfft_amd_execute_static
STATIC_WORK_BYTES = 64 << 20

EXPORTED_SYMBOLS = tuple(_PROTOTYPES)


class Library:
    """One loaded copy of the shared library."""

    def __init__(self, path=None, extensions=True):
        """extensions=False loads any library that speaks rocfft.h (the reference's own
        librocfft.so, to time it through the same calls): the rocfft_amd_* entry points are
        then not looked up."""
        path = path or library_path()
        if not os.path.exists(path):
            raise FileNotFoundError(
                "%s is missing: build it with __graft_entry__.build() (hipcc, gfx950); "
                "there is no fallback implementation" % path)
        self.path = path
        self.extensions = extensions
        # PyTorch wheels carry their own copy of the HIP runtime under the same soname.
        # When a process uses both, torch must be loaded first so that this library
        # binds to the runtime torch initialises (one runtime per process).
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        self.c = ctypes.CDLL(path)
        for name, args in _PROTOTYPES.items():
            if not extensions and name.startswith("rocfft_amd_"):
                continue
            fn = getattr(self.c, name)
            fn.argtypes = args
            fn.restype = ctypes.c_int

    def check(self, status, what):
        if status != STATUS_SUCCESS:
            raise RocfftError(status, what)

    def setup(self):
        self.check(self.c.rocfft_setup(), "rocfft_setup")

    def cleanup(self):
        self.check(self.c.rocfft_cleanup(), "rocfft_cleanup")

    def version(self):
        buf = ctypes.create_string_buffer(64)
        self.check(self.c.rocfft_get_version_string(buf, 64), "rocfft_get_version_string")
        return buf.value.decode()

    def copy_probe(self, stream=None, **fields):
        """enqueues one copy probe (rocfft_amd_copy_probe) on `stream`"""
        q = Probe(**fields)
        self.check(self.c.rocfft_amd_copy_probe(ctypes.byref(q), stream), "rocfft_amd_copy_probe")

    def describe(self, placement, transform_type, precision, lengths, batch=1, description=None):
        """Plan text and work-buffer bytes without touching a device."""
        ln = (ctypes.c_size_t * len(lengths))(*lengths)
        text = ctypes.create_string_buffer(1 << 16)
        work = ctypes.c_size_t(0)
        st = self.c.rocfft_amd_plan_describe(placement, transform_type, precision, len(lengths), ln,
                                             batch, description.handle if description else None,
                                             text, len(text), ctypes.byref(work))
        return st, text.value.decode(), work.value


_DEFAULT = None


def library():
    """The product library (loaded once)."""
    global _DEFAULT
    if _DEFAULT is None:
        _DEFAULT = Library()
        _DEFAULT.setup()
    return _DEFAULT


def _size_array(values):
    if values is None:
        return None
    return (ctypes.c_size_t * len(values))(*[int(v) for v in values])


class PlanDescription:
    def __init__(self, lib=None):
        self.lib = lib or library()
        h = ctypes.c_void_p()
        self.lib.check(self.lib.c.rocfft_plan_description_create(ctypes.byref(h)),
                       "rocfft_plan_description_create")
        self.handle = h

    def set_data_layout(self, in_array_type, out_array_type, in_offsets=None, out_offsets=None,
                        in_strides=None, in_distance=0, out_strides=None, out_distance=0):
        st = self.lib.c.rocfft_plan_description_set_data_layout(
            self.handle, in_array_type, out_array_type, _size_array(in_offsets),
            _size_array(out_offsets), len(in_strides) if in_strides else 0, _size_array(in_strides),
            in_distance, len(out_strides) if out_strides else 0, _size_array(out_strides),
            out_distance)
        self.lib.check(st, "rocfft_plan_description_set_data_layout")
        return self

    def set_scale_factor(self, scale):
        st = self.lib.c.rocfft_plan_description_set_scale_factor(self.handle, float(scale))
        self.lib.check(st, "rocfft_plan_description_set_scale_factor")
        return self

    def destroy(self):
        if self.handle:
            self.lib.c.rocfft_plan_description_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class ExecutionInfo:
    def __init__(self, lib=None):
        self.lib = lib or library()
        h = ctypes.c_void_p()
        self.lib.check(self.lib.c.rocfft_execution_info_create(ctypes.byref(h)),
                       "rocfft_execution_info_create")
        self.handle = h

    def set_work_buffer(self, ptr, size_in_bytes):
        st = self.lib.c.rocfft_execution_info_set_work_buffer(self.handle, ctypes.c_void_p(ptr),
                                                              size_in_bytes)
        self.lib.check(st, "rocfft_execution_info_set_work_buffer")
        return self

    def set_stream(self, stream):
        st = self.lib.c.rocfft_execution_info_set_stream(self.handle, ctypes.c_void_p(stream))
        self.lib.check(st, "rocfft_execution_info_set_stream")
        return self

    def _set_callback(self, name, fn, data, shared_mem_bytes):
        fns = (ctypes.c_void_p * 1)(fn)
        datas = (ctypes.c_void_p * 1)(data)
        return getattr(self.lib.c, name)(self.handle, fns, datas, shared_mem_bytes)

    def set_load_callback(self, fn, data=None, shared_mem_bytes=0):
        """fn: device address of `T load_cb(T* data, size_t offset, void* cbdata, void* sharedMem)`
        (None clears it); data: the cbdata pointer"""
        st = self._set_callback("rocfft_execution_info_set_load_callback", fn, data, shared_mem_bytes)
        self.lib.check(st, "rocfft_execution_info_set_load_callback")
        return self

    def set_store_callback(self, fn, data=None, shared_mem_bytes=0):
        """fn: device address of `void store_cb(T* data, size_t offset, T element, void* cbdata,
        void* sharedMem)` (None clears it)"""
        st = self._set_callback("rocfft_execution_info_set_store_callback", fn, data, shared_mem_bytes)
        self.lib.check(st, "rocfft_execution_info_set_store_callback")
        return self

    def destroy(self):
        if self.handle:
            self.lib.c.rocfft_execution_info_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class Plan:
    def __init__(self, placement, transform_type, precision, lengths, batch=1, description=None,
                 lib=None):
        self.lib = lib or library()
        self.lengths = [int(v) for v in lengths]
        self.batch = int(batch)
        h = ctypes.c_void_p()
        st = self.lib.c.rocfft_plan_create(ctypes.byref(h), placement, transform_type, precision,
                                           len(self.lengths), _size_array(self.lengths), self.batch,
                                           description.handle if description else None)
        self.lib.check(st, "rocfft_plan_create")
        self.handle = h

    @property
    def work_buffer_size(self):
        n = ctypes.c_size_t(0)
        self.lib.check(self.lib.c.rocfft_plan_get_work_buffer_size(self.handle, ctypes.byref(n)),
                       "rocfft_plan_get_work_buffer_size")
        return n.value

    def print(self):
        self.lib.check(self.lib.c.rocfft_plan_get_print(self.handle), "rocfft_plan_get_print")

    def execute_status(self, in_ptrs, out_ptrs=None, info=None):
        ins = (ctypes.c_void_p * 2)(*(list(in_ptrs) + [None])[:2])
        outs = None
        if out_ptrs is not None:
            outs = (ctypes.c_void_p * 2)(*(list(out_ptrs) + [None])[:2])
        return self.lib.c.rocfft_execute(self.handle, ins, outs, info.handle if info else None)

    def execute(self, in_ptrs, out_ptrs=None, info=None):
        self.lib.check(self.execute_status(in_ptrs, out_ptrs, info), "rocfft_execute")

    def execute_static_status(self, in_ptrs, out_ptrs=None, info=None):
        """rocfft_amd_execute_static: the work area is the library's own static device array"""
        ins = (ctypes.c_void_p * 2)(*(list(in_ptrs) + [None])[:2])
        outs = None
        if out_ptrs is not None:
            outs = (ctypes.c_void_p * 2)(*(list(out_ptrs) + [None])[:2])
        return self.lib.c.rocfft_amd_execute_static(self.handle, ins, outs, info.handle if info else None)

    def execute_static(self, in_ptrs, out_ptrs=None, info=None):
        self.lib.check(self.execute_static_status(in_ptrs, out_ptrs, info), "rocfft_amd_execute_static")

    def passes(self):
        """[(name, bytes read + written)] of the plan's kernel launches, in order"""
        n = ctypes.c_size_t(0)
        self.lib.check(self.lib.c.rocfft_amd_plan_get_pass_count(self.handle, ctypes.byref(n)),
                       "rocfft_amd_plan_get_pass_count")
        out = []
        for i in range(n.value):
            name = ctypes.create_string_buffer(256)
            nbytes = ctypes.c_double(0)
            self.lib.check(self.lib.c.rocfft_amd_plan_get_pass_info(self.handle, i, name, 256,
                                                                    ctypes.byref(nbytes)),
                           "rocfft_amd_plan_get_pass_info")
            out.append((name.value.decode(), nbytes.value))
        return out

    def execute_profile(self, in_ptrs, out_ptrs=None, info=None):
        """like execute, but waits and returns the duration of every pass in milliseconds"""
        npass = len(self.passes())
        ms = (ctypes.c_float * max(npass, 1))()
        ins = (ctypes.c_void_p * 2)(*(list(in_ptrs) + [None])[:2])
        outs = None
        if out_ptrs is not None:
            outs = (ctypes.c_void_p * 2)(*(list(out_ptrs) + [None])[:2])
        st = self.lib.c.rocfft_amd_execute_profile(self.handle, ins, outs, info.handle if info else None,
                                                   ms, npass)
        self.lib.check(st, "rocfft_amd_execute_profile")
        return [ms[i] for i in range(npass)]

    def destroy(self):
        if self.handle:
            self.lib.c.rocfft_plan_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
