"""ctypes wrapper of oracle/sched_ref.c (the scheduler oracle) -- TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libsched_ref.so")


class _State(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in ("max_requests", "max_tokens", "max_pages", "page_size", "max_seq", "max_new_per_req", "total_requests")] + \
               [("eos_token_id", ctypes.c_int64)] + \
               [(n, ctypes.c_void_p) for n in ("step", "tokens", "input_tokens", "output_tokens", "prompt_lengths", "qo_indptr", "kv_indptr",
                                               "kv_indices", "kv_last_page_len", "request_ids", "page_queue")] + \
               [(n, ctypes.c_int32) for n in ("page_queue_head", "page_queue_tail", "next_request_id")]


def _load():
    if not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(os.path.join(_HERE, "sched_ref.c")):
        subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    lib = ctypes.CDLL(_LIB)
    lib.sched_ref_reset.argtypes = [ctypes.POINTER(_State)]
    lib.sched_ref_prepare_next_batch.argtypes = [ctypes.POINTER(_State)]
    lib.sched_ref_prepare_next_batch.restype = ctypes.c_int
    return lib


class SchedulerOracle:
    """Holds numpy copies of the meta tensors and steps the C oracle over them."""

    def __init__(self, prompts, max_requests, max_tokens, max_pages, page_size, max_seq, eos=0x7FFFFFFF, max_new_per_req=8):
        self.lib = _load()
        T = len(prompts)
        self.a = {
            "step": np.zeros(T, np.int32), "tokens": np.zeros((T, max_seq), np.int64), "input_tokens": np.zeros(max_tokens, np.int64),
            "output_tokens": np.zeros(max_tokens, np.int64), "prompt_lengths": np.array([len(p) for p in prompts], np.int32),
            "qo_indptr": np.zeros(max_requests + 1, np.int32), "kv_indptr": np.zeros(max_requests + 1, np.int32),
            "kv_indices": np.zeros(max_pages, np.int32), "kv_last_page_len": np.zeros(max_requests, np.int32),
            "request_ids": np.zeros(max_requests, np.int32), "page_queue": np.zeros(max_pages, np.int32)}
        for r, p in enumerate(prompts):
            self.a["tokens"][r, :len(p)] = np.asarray(p, np.int64)
        s = _State()
        s.max_requests, s.max_tokens, s.max_pages, s.page_size, s.max_seq = max_requests, max_tokens, max_pages, page_size, max_seq
        s.max_new_per_req, s.total_requests, s.eos_token_id = max_new_per_req, T, eos
        for k, v in self.a.items():
            setattr(s, k, v.ctypes.data)
        self.s = s
        self.lib.sched_ref_reset(ctypes.byref(s))

    def step(self, output_tokens=None):
        """Feed the tokens the model produced for the current batch rows and schedule the next batch."""
        if output_tokens is not None:
            self.a["output_tokens"][:len(output_tokens)] = np.asarray(output_tokens, np.int64)
        return int(self.lib.sched_ref_prepare_next_batch(ctypes.byref(self.s)))

    def __getitem__(self, k):
        return self.a[k]

    @property
    def free_pages(self):
        return int(self.s.page_queue_tail - self.s.page_queue_head)
