"""ctypes binding of libfleet_mk.so (declared in include/fleet_mk.h).

Takes the place of the reference's Cython module (python/mirage/_cython/core.pyx) for the
decode path.  There is no CPU fallback: if the shared library is missing the import of any
compute entry point raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# FLEET_MK_LIB selects another build of the same library (used to compare tuning variants)
LIB_PATH = os.environ.get("FLEET_MK_LIB") or os.path.join(os.path.dirname(_HERE), "libfleet_mk.so")

MK_OK = 0
MK_EINVAL = -1
MK_EHIP = -2
MK_ESTATE = -3
MK_EABORT = -4
MK_EUNSUPPORTED = -5

MK_CFG_SINGLE_WEIGHT_COPY = 1
MK_MODES = {"offline": 0, "online": 1, "online_notoken": 2, "onepass": 3}

# symbols include/fleet_mk.h declares; tests check that the library exports every one
EXPORTED_SYMBOLS = [
    "mk_graph_create", "mk_graph_destroy", "mk_tensor_attach", "mk_tensor_new", "mk_tensor_shuffle",
    "mk_tensor_num_dims", "mk_tensor_dim", "mk_tensor_ptr", "mk_add_task", "mk_generate_task_graph",
    "mk_compile", "mk_init_requests", "mk_launch", "mk_launch_steps", "mk_enqueue_steps", "mk_enqueue_steps_static", "mk_wait",
    "mk_run_once", "mk_repack_weights", "mk_tensor_releasable", "mk_set_profiler", "mk_get_stats", "mk_get_stage_profile", "mk_get_stage_marks", "mk_describe_program", "mk_last_error", "mk_version",
]


class MkConfig(ctypes.Structure):
    _fields_ = [
        ("num_workers", ctypes.c_int),
        ("max_seq_length", ctypes.c_int),
        ("max_num_batched_requests", ctypes.c_int),
        ("max_num_batched_tokens", ctypes.c_int),
        ("max_num_pages", ctypes.c_int),
        ("page_size", ctypes.c_int),
        ("total_num_requests", ctypes.c_int),
        ("device", ctypes.c_int),
        ("eos_token_id", ctypes.c_int64),
        ("rms_eps", ctypes.c_float),
        ("mode", ctypes.c_int),
        ("max_tokens_per_request", ctypes.c_int),
        ("flags", ctypes.c_int),
        ("step", ctypes.c_void_p),
        ("tokens", ctypes.c_void_p),
        ("input_tokens", ctypes.c_void_p),
        ("output_tokens", ctypes.c_void_p),
        ("num_new_tokens", ctypes.c_void_p),
        ("prompt_lengths", ctypes.c_void_p),
        ("qo_indptr", ctypes.c_void_p),
        ("paged_kv_indptr", ctypes.c_void_p),
        ("paged_kv_indices", ctypes.c_void_p),
        ("paged_kv_last_page_len", ctypes.c_void_p),
    ]


class MkStats(ctypes.Structure):
    _fields_ = [
        ("num_workgroups", ctypes.c_int),
        ("num_stages", ctypes.c_int),
        ("num_tasks", ctypes.c_int),
        ("num_events", ctypes.c_int),
        ("num_xcds", ctypes.c_int),
        ("aborted", ctypes.c_int),
        ("iterations", ctypes.c_int64),
        ("weight_bytes", ctypes.c_int64),
        ("last_launch_ms", ctypes.c_double),
        ("packed_weight_bytes", ctypes.c_int64),
        ("row_major_weight_bytes", ctypes.c_int64),
    ]


class MkError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"fleet_mk error {code}: {message}")
        self.code = code
        self.message = message


_lib = None


def load():
    """Load libfleet_mk.so; raises if it has not been built (python fleet-chiplet-megakernel_amd/build.py)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: build it with `python fleet-chiplet-megakernel_amd/build.py` "
            "(the decode megakernel has no CPU fallback)")
    lib = ctypes.CDLL(LIB_PATH)
    vp, ci, cip = ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_int)
    i64p = ctypes.POINTER(ctypes.c_int64)
    lib.mk_graph_create.argtypes = [ctypes.POINTER(MkConfig), ctypes.POINTER(vp)]
    lib.mk_graph_destroy.argtypes = [vp]
    lib.mk_tensor_attach.argtypes = [vp, vp, ci, i64p, i64p, ci, ctypes.c_char_p]
    lib.mk_tensor_new.argtypes = [vp, ci, i64p, i64p, ci, ctypes.c_char_p, ci]
    lib.mk_tensor_shuffle.argtypes = [vp, cip, ci, ci, ci, ci, ctypes.c_char_p]
    lib.mk_tensor_num_dims.argtypes = [vp, ci]
    lib.mk_tensor_dim.argtypes = [vp, ci, ci]
    lib.mk_tensor_dim.restype = ctypes.c_int64
    lib.mk_tensor_ptr.argtypes = [vp, ci]
    lib.mk_tensor_ptr.restype = vp
    lib.mk_add_task.argtypes = [vp, ctypes.c_char_p, cip, cip, ci, cip, cip, cip, ci, cip]
    lib.mk_generate_task_graph.argtypes = [vp, ci, ci, ctypes.POINTER(ctypes.c_char_p)]
    lib.mk_compile.argtypes = [vp]
    lib.mk_init_requests.argtypes = [vp]
    lib.mk_launch.argtypes = [vp, vp]
    lib.mk_launch_steps.argtypes = [vp, vp, ci, cip]
    lib.mk_enqueue_steps.argtypes = [vp, vp, ci]
    lib.mk_enqueue_steps_static.argtypes = [vp, vp, ci]
    lib.mk_wait.argtypes = [vp, vp, cip]
    i32p = ctypes.POINTER(ctypes.c_int32)
    lib.mk_run_once.argtypes = [vp, vp, ci, i32p, i32p, i32p]
    lib.mk_get_stats.argtypes = [vp, ctypes.POINTER(MkStats)]
    lib.mk_get_stage_profile.argtypes = [vp, ci, ctypes.POINTER(ctypes.c_int64), ci]
    lib.mk_repack_weights.argtypes = [vp]
    lib.mk_tensor_releasable.argtypes = [vp, ci]
    lib.mk_set_profiler.argtypes = [vp, vp, ctypes.c_int64]
    lib.mk_get_stage_marks.argtypes = [vp, ci, ctypes.POINTER(ctypes.c_int64), ci]
    lib.mk_describe_program.argtypes = [vp, ctypes.POINTER(ctypes.c_char_p)]
    lib.mk_last_error.restype = ctypes.c_char_p
    lib.mk_version.restype = ctypes.c_char_p
    _lib = lib
    return lib


def check(rc):
    """Raise MkError for a negative status; pass non-negative values (ids) through."""
    if rc < 0:
        raise MkError(rc, load().mk_last_error().decode())
    return rc


def int_array(values, ctype=ctypes.c_int):
    values = list(values)
    return (ctype * max(1, len(values)))(*values)


CONFIG_FIELDS = [name for name, _ in MkConfig._fields_]
STATS_FIELDS = [name for name, _ in MkStats._fields_]


class Graph:
    """One mk_graph handle behind plain-Python methods (ints, sequences, bytes in; ints, str, dict out; MkError on a
    negative status).  This is the ctypes implementation; `mirage._cython.core.CyGraph` is the same interface compiled
    with Cython against include/fleet_mk.h (what the reference's `CyKNGraph` / launcher module are to its C++ graph,
    python/mirage/_cython/core.pyx).  `make_graph` picks one."""
    binding = "ctypes"

    def __init__(self, cfg: dict):
        self._lib = load()
        c = MkConfig()
        for k, v in cfg.items():
            if k not in CONFIG_FIELDS:
                raise KeyError(f"mk_config has no field '{k}'")
            setattr(c, k, v)
        h = ctypes.c_void_p()
        check(self._lib.mk_graph_create(ctypes.byref(c), ctypes.byref(h)))
        self._h = h

    @property
    def handle(self) -> int:
        """Address of the mk_graph (for callers that talk to the C ABI directly)."""
        return self._h.value or 0

    def tensor_attach(self, ptr, dims, strides, dtype_code, name):
        return check(self._lib.mk_tensor_attach(self._h, ctypes.c_void_p(ptr), len(dims), int_array(dims, ctypes.c_int64),
                                                int_array(strides, ctypes.c_int64), dtype_code, name.encode()))

    def tensor_new(self, dims, strides, dtype_code, name, io_category):
        sp = int_array(strides, ctypes.c_int64) if strides is not None else None
        return check(self._lib.mk_tensor_new(self._h, len(dims), int_array(dims, ctypes.c_int64), sp, dtype_code, name.encode(), io_category))

    def tensor_shuffle(self, ids, dim, num_groups, interleave, name):
        return check(self._lib.mk_tensor_shuffle(self._h, int_array(ids), len(ids), dim, num_groups, 1 if interleave else 0, name.encode()))

    def tensor_ptr(self, tid) -> int:
        return self._lib.mk_tensor_ptr(self._h, tid) or 0

    def tensor_releasable(self, tid) -> bool:
        return check(self._lib.mk_tensor_releasable(self._h, tid)) == 1

    def add_task(self, name, grid_dim, block_dim, tensor_ids, input_maps, forloop_dims, params):
        check(self._lib.mk_add_task(self._h, name.encode(), int_array(grid_dim), int_array(block_dim), len(tensor_ids), int_array(tensor_ids),
                                    int_array(input_maps), int_array(forloop_dims), len(params), int_array(params)))

    def generate_task_graph(self, num_gpus, my_gpu_id) -> str:
        out = ctypes.c_char_p()
        check(self._lib.mk_generate_task_graph(self._h, num_gpus, my_gpu_id, ctypes.byref(out)))
        return out.value.decode()

    def describe_program(self) -> str:
        out = ctypes.c_char_p()
        check(self._lib.mk_describe_program(self._h, ctypes.byref(out)))
        return out.value.decode()

    def compile(self):
        check(self._lib.mk_compile(self._h))

    def init_requests(self):
        check(self._lib.mk_init_requests(self._h))

    def set_profiler(self, ptr, num_entries):
        check(self._lib.mk_set_profiler(self._h, ctypes.c_void_p(ptr) if ptr else None, num_entries))

    def launch(self, stream):
        check(self._lib.mk_launch(self._h, ctypes.c_void_p(stream)))

    def launch_steps(self, stream, max_iterations) -> bool:
        fin = ctypes.c_int(0)
        check(self._lib.mk_launch_steps(self._h, ctypes.c_void_p(stream), int(max_iterations), ctypes.byref(fin)))
        return bool(fin.value)

    def enqueue_steps(self, stream, max_iterations, static=False):
        fn = self._lib.mk_enqueue_steps_static if static else self._lib.mk_enqueue_steps
        check(fn(self._h, ctypes.c_void_p(stream), int(max_iterations)))

    def wait(self, stream) -> bool:
        fin = ctypes.c_int(0)
        check(self._lib.mk_wait(self._h, ctypes.c_void_p(stream), ctypes.byref(fin)))
        return bool(fin.value)

    def run_once(self, stream, tok_slot, tok_pos, tok_first):
        i32 = ctypes.c_int32
        check(self._lib.mk_run_once(self._h, ctypes.c_void_p(stream), len(tok_slot), int_array(tok_slot, i32), int_array(tok_pos, i32),
                                    int_array(tok_first, i32)))

    def repack_weights(self):
        check(self._lib.mk_repack_weights(self._h))

    def stats(self) -> dict:
        st = MkStats()
        check(self._lib.mk_get_stats(self._h, ctypes.byref(st)))
        return {name: getattr(st, name) for name in STATS_FIELDS}

    def stage_ticks(self, workgroup, max_stages, marks=False) -> list:
        """Rows of four 100 MHz ticks per stage (mk_get_stage_profile, or mk_get_stage_marks)."""
        buf = (ctypes.c_int64 * (4 * max_stages))()
        fn = self._lib.mk_get_stage_marks if marks else self._lib.mk_get_stage_profile
        got = check(fn(self._h, int(workgroup), buf, max_stages))
        return [[int(buf[4 * i + k]) for k in range(4)] for i in range(got)]

    def destroy(self):
        if self._h is not None and self._h.value:
            self._lib.mk_graph_destroy(self._h)
        self._h = None


def make_graph(cfg: dict, binding: str = None):
    """A graph handle through the binding named by `binding` or FLEET_MK_BINDING: "ctypes" (default, needs no build step
    beyond the library) or "cython" (the compiled shim; `python fleet-chiplet-megakernel_amd/build.py` builds it)."""
    binding = binding or os.environ.get("FLEET_MK_BINDING", "ctypes")
    if binding == "ctypes":
        return Graph(cfg)
    if binding == "cython":
        load()  # the shim links against the same library: make sure it is there, with the usual message if not
        try:
            from ._cython import core
        except ImportError as e:
            raise ImportError(f"the Cython binding is not built ({e}); run `python fleet-chiplet-megakernel_amd/build.py`") from None
        return core.CyGraph(cfg)
    raise ValueError(f"unknown binding '{binding}' (ctypes or cython)")


def load_address():
    """Address at which the shared library is mapped in this process (0 if it cannot be determined): lets a crash report
    that lists program counters be matched against the library."""
    load()
    try:
        with open("/proc/self/maps") as f:
            for line in f:
                if line.rstrip().endswith(os.path.basename(LIB_PATH)):
                    return int(line.split("-", 1)[0], 16)
    except OSError:
        pass
    return 0
