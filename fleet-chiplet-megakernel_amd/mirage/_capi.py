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
