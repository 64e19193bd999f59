# cython: language_level=3
"""Compiled binding of libfleet_mk.so.  `CyGraph` owns one mk_graph handle and offers the interface of
`mirage._capi.Graph` (plain Python values in and out, MkError on a negative status); select it with
FLEET_MK_BINDING=cython or `mirage._capi.make_graph(cfg, "cython")`.

What the reference's Cython layer does for its C++ graph (python/mirage/_cython/core.pyx: CyKNGraph.new_input /
attach_torch_tensor / register_task / generate_task_graph, and the launcher module's init_func / launch_func /
finalize_func, python/mirage/mpk/persistent_kernel.py:63-68,2600-2658) maps onto the methods below one to one."""
from libc.stdint cimport int32_t, int64_t, uintptr_t
from libc.stdlib cimport malloc, free
cimport fleet_mk as mk

from .._capi import MkError


cdef int _check(int rc) except? -1000000:
    if rc < 0:
        raise MkError(rc, (<bytes>mk.mk_last_error()).decode())
    return rc


cdef int *_ints(seq, int *n) except NULL:
    """A malloc'ed int array holding `seq` (at least one element, so that the pointer is never NULL)."""
    cdef Py_ssize_t i, k = len(seq)
    cdef int *a = <int *>malloc(sizeof(int) * (k if k > 0 else 1))
    if a == NULL:
        raise MemoryError()
    for i in range(k):
        a[i] = <int>seq[i]
    n[0] = <int>k
    return a


cdef int64_t *_longs(seq, int *n) except NULL:
    cdef Py_ssize_t i, k = len(seq)
    cdef int64_t *a = <int64_t *>malloc(sizeof(int64_t) * (k if k > 0 else 1))
    if a == NULL:
        raise MemoryError()
    for i in range(k):
        a[i] = <int64_t>seq[i]
    n[0] = <int>k
    return a


def version() -> str:
    return (<bytes>mk.mk_version()).decode()


cdef class CyGraph:
    cdef mk.mk_graph *g
    binding = "cython"

    def __cinit__(self, dict cfg):
        cdef mk.mk_config c
        self.g = NULL
        known = ("num_workers", "max_seq_length", "max_num_batched_requests", "max_num_batched_tokens", "max_num_pages", "page_size",
                 "total_num_requests", "device", "eos_token_id", "rms_eps", "mode", "max_tokens_per_request", "flags", "step", "tokens",
                 "input_tokens", "output_tokens", "num_new_tokens", "prompt_lengths", "qo_indptr", "paged_kv_indptr", "paged_kv_indices",
                 "paged_kv_last_page_len")
        for k in cfg:
            if k not in known:
                raise KeyError(f"mk_config has no field '{k}'")
        g = cfg.get
        c.num_workers = g("num_workers", 0)
        c.max_seq_length = g("max_seq_length", 0)
        c.max_num_batched_requests = g("max_num_batched_requests", 0)
        c.max_num_batched_tokens = g("max_num_batched_tokens", 0)
        c.max_num_pages = g("max_num_pages", 0)
        c.page_size = g("page_size", 0)
        c.total_num_requests = g("total_num_requests", 0)
        c.device = g("device", 0)
        c.eos_token_id = g("eos_token_id", 0)
        c.rms_eps = g("rms_eps", 0.0)
        c.mode = g("mode", 0)
        c.max_tokens_per_request = g("max_tokens_per_request", 0)
        c.flags = g("flags", 0)
        c.step = <int32_t *><uintptr_t>(g("step", 0) or 0)
        c.tokens = <int64_t *><uintptr_t>(g("tokens", 0) or 0)
        c.input_tokens = <int64_t *><uintptr_t>(g("input_tokens", 0) or 0)
        c.output_tokens = <int64_t *><uintptr_t>(g("output_tokens", 0) or 0)
        c.num_new_tokens = <int32_t *><uintptr_t>(g("num_new_tokens", 0) or 0)
        c.prompt_lengths = <int32_t *><uintptr_t>(g("prompt_lengths", 0) or 0)
        c.qo_indptr = <int32_t *><uintptr_t>(g("qo_indptr", 0) or 0)
        c.paged_kv_indptr = <int32_t *><uintptr_t>(g("paged_kv_indptr", 0) or 0)
        c.paged_kv_indices = <int32_t *><uintptr_t>(g("paged_kv_indices", 0) or 0)
        c.paged_kv_last_page_len = <int32_t *><uintptr_t>(g("paged_kv_last_page_len", 0) or 0)
        _check(mk.mk_graph_create(&c, &self.g))

    def __dealloc__(self):
        if self.g != NULL:
            mk.mk_graph_destroy(self.g)
            self.g = NULL

    @property
    def handle(self) -> int:
        return <uintptr_t>self.g

    # ---- tensors (CyKNGraph.new_input + attach_torch_tensor / attach_cuda_tensor, core.pyx:718,944-965)
    def tensor_attach(self, ptr, dims, strides, int dtype_code, str name):
        cdef int nd = 0, ns = 0
        cdef int64_t *d = _longs(dims, &nd)
        cdef int64_t *s = _longs(strides, &ns)
        nm = name.encode()
        try:
            return _check(mk.mk_tensor_attach(self.g, <void *><uintptr_t>(ptr or 0), nd, d, s, dtype_code, nm))
        finally:
            free(d)
            free(s)

    def tensor_new(self, dims, strides, int dtype_code, str name, int io_category):
        cdef int nd = 0, ns = 0
        cdef int64_t *d = _longs(dims, &nd)
        cdef int64_t *s = NULL
        if strides is not None:
            s = _longs(strides, &ns)
        nm = name.encode()
        try:
            return _check(mk.mk_tensor_new(self.g, nd, d, s, dtype_code, nm, io_category))
        finally:
            free(d)
            if s != NULL:
                free(s)

    def tensor_shuffle(self, ids, int dim, int num_groups, interleave, str name):
        cdef int n = 0
        cdef int *a = _ints(ids, &n)
        nm = name.encode()
        try:
            return _check(mk.mk_tensor_shuffle(self.g, a, n, dim, num_groups, 1 if interleave else 0, nm))
        finally:
            free(a)

    def tensor_ptr(self, int tid) -> int:
        return <uintptr_t>mk.mk_tensor_ptr(self.g, tid)

    def tensor_releasable(self, int tid) -> bool:
        return _check(mk.mk_tensor_releasable(self.g, tid)) == 1

    # ---- tasks (TBGraph.new_input per operand + KNGraph.customized + register_task, core.pyx:817,1011-1059)
    def add_task(self, str name, grid_dim, block_dim, tensor_ids, input_maps, forloop_dims, params):
        cdef int n3 = 0, nops = 0, nmaps = 0, nfl = 0, npar = 0
        cdef int *gd = _ints(grid_dim, &n3)
        cdef int *bd = _ints(block_dim, &n3)
        cdef int *ids = _ints(tensor_ids, &nops)
        cdef int *maps = _ints(input_maps, &nmaps)
        cdef int *fl = _ints(forloop_dims, &nfl)
        cdef int *par = _ints(params, &npar)
        nm = name.encode()
        try:
            if len(grid_dim) != 3 or len(block_dim) != 3 or nmaps != 3 * nops or nfl != nops:
                raise ValueError("add_task: grid and block have three entries, every operand three map entries and one loop dim")
            _check(mk.mk_add_task(self.g, nm, gd, bd, nops, ids, maps, fl, npar, par))
        finally:
            free(gd)
            free(bd)
            free(ids)
            free(maps)
            free(fl)
            free(par)

    def generate_task_graph(self, int num_gpus, int my_gpu_id) -> str:
        cdef const char *out = NULL
        _check(mk.mk_generate_task_graph(self.g, num_gpus, my_gpu_id, &out))
        return (<bytes>out).decode()

    def describe_program(self) -> str:
        cdef const char *out = NULL
        _check(mk.mk_describe_program(self.g, &out))
        return (<bytes>out).decode()

    # ---- launcher (init_func / launch_func / finalize_func of the reference's generated module)
    def compile(self):
        cdef int rc
        with nogil:
            rc = mk.mk_compile(self.g)
        _check(rc)

    def init_requests(self):
        _check(mk.mk_init_requests(self.g))

    def set_profiler(self, ptr, num_entries):
        _check(mk.mk_set_profiler(self.g, <void *><uintptr_t>(ptr or 0), <int64_t>num_entries))

    def launch(self, stream):
        cdef int rc
        cdef void *s = <void *><uintptr_t>(stream or 0)
        with nogil:
            rc = mk.mk_launch(self.g, s)
        _check(rc)

    def launch_steps(self, stream, int max_iterations) -> bool:
        cdef int rc, fin = 0
        cdef void *s = <void *><uintptr_t>(stream or 0)
        with nogil:
            rc = mk.mk_launch_steps(self.g, s, max_iterations, &fin)
        _check(rc)
        return fin != 0

    def enqueue_steps(self, stream, int max_iterations, static=False):
        cdef void *s = <void *><uintptr_t>(stream or 0)
        if static:
            _check(mk.mk_enqueue_steps_static(self.g, s, max_iterations))
        else:
            _check(mk.mk_enqueue_steps(self.g, s, max_iterations))

    def wait(self, stream) -> bool:
        cdef int rc, fin = 0
        cdef void *s = <void *><uintptr_t>(stream or 0)
        with nogil:
            rc = mk.mk_wait(self.g, s, &fin)
        _check(rc)
        return fin != 0

    def run_once(self, stream, tok_slot, tok_pos, tok_first):
        cdef int n = 0, n2 = 0, n3 = 0
        cdef int *a = _ints(tok_slot, &n)
        cdef int *b = _ints(tok_pos, &n2)
        cdef int *c = _ints(tok_first, &n3)
        try:
            if n2 != n or n3 != n:
                raise ValueError("run_once: one slot, position and first-row index per token row")
            _check(mk.mk_run_once(self.g, <void *><uintptr_t>(stream or 0), n, <const int32_t *>a, <const int32_t *>b, <const int32_t *>c))
        finally:
            free(a)
            free(b)
            free(c)

    def repack_weights(self):
        _check(mk.mk_repack_weights(self.g))

    def stats(self) -> dict:
        cdef mk.mk_stats st
        _check(mk.mk_get_stats(self.g, &st))
        return {"num_workgroups": st.num_workgroups, "num_stages": st.num_stages, "num_tasks": st.num_tasks, "num_events": st.num_events,
                "num_xcds": st.num_xcds, "aborted": st.aborted, "iterations": st.iterations, "weight_bytes": st.weight_bytes,
                "last_launch_ms": st.last_launch_ms, "packed_weight_bytes": st.packed_weight_bytes,
                "row_major_weight_bytes": st.row_major_weight_bytes}

    def stage_ticks(self, int workgroup, int max_stages, marks=False) -> list:
        cdef int64_t *buf = <int64_t *>malloc(sizeof(int64_t) * 4 * (max_stages if max_stages > 0 else 1))
        cdef int got, i, k
        if buf == NULL:
            raise MemoryError()
        try:
            if marks:
                got = _check(mk.mk_get_stage_marks(self.g, workgroup, buf, max_stages))
            else:
                got = _check(mk.mk_get_stage_profile(self.g, workgroup, buf, max_stages))
            return [[buf[4 * i + k] for k in range(4)] for i in range(got)]
        finally:
            free(buf)

    def destroy(self):
        if self.g != NULL:
            mk.mk_graph_destroy(self.g)
            self.g = NULL
