"""Graph-side objects of the PersistentKernel API: dtypes, DTensor handles and the KNGraph facade.

Mirrors the parts of python/mirage/kernel.py and python/mirage/_cython/core.pyx (DTensor.dim /
num_dims, core.pyx:431-482; KNGraph.generate_task_graph, kernel.py) that demo/qwen3/demo.py touches.
The graph itself lives behind the C ABI (include/fleet_mk.h).
"""
import ctypes

import torch

from . import _capi


class dtype:
    """Element type tag; `code` is the reference's type::DataType value (include/mirage/type.h:58-73)."""

    def __init__(self, name, code, torch_dtype, size):
        self.name, self.code, self.torch_dtype, self.size = name, code, torch_dtype, size

    def __repr__(self):
        return f"mirage.{self.name}"


float16 = dtype("float16", 940, torch.float16, 2)
bfloat16 = dtype("bfloat16", 941, torch.bfloat16, 2)
float32 = dtype("float32", 950, torch.float32, 4)
int32 = dtype("int32", 955, torch.int32, 4)
int64 = dtype("int64", 965, torch.int64, 8)
uint64 = dtype("uint64", 966, torch.uint64, 8)

_ALL = [float16, bfloat16, float32, int32, int64, uint64]


def convert_torch_type_to_dtype(t):
    for d in _ALL:
        if d.torch_dtype == t:
            return d
    raise RuntimeError(f"Unsupported torch dtype {t}")


def convert_dtype_to_torch_type(d):
    return d.torch_dtype


class DTensor:
    """Handle to a device tensor recorded in the graph (core.pyx:431-482)."""

    def __init__(self, graph, tid, dims, dt, name, torch_tensor=None):
        self._graph = graph
        self.id = tid
        self._dims = tuple(int(d) for d in dims)
        self.dtype = dt
        self.name = name
        self.torch_tensor = torch_tensor  # keeps attached storage alive as long as the handle

    @property
    def num_dims(self):
        return len(self._dims)

    def dim(self, i):
        if i < 0 or i >= len(self._dims):
            raise IndexError(f"dim {i} out of range for tensor with {len(self._dims)} dims")
        return self._dims[i]

    @property
    def shape(self):
        return self._dims

    def data_ptr(self):
        return self._graph._g.tensor_ptr(self.id) or None

    def to_torch(self):
        """A torch view of this tensor's device memory (library-owned tensors included)."""
        if self.torch_tensor is not None:
            return self.torch_tensor
        return self._graph._torch_view(self)

    def __repr__(self):
        return f"DTensor({self.name}, dims={self._dims}, {self.dtype})"


class KNGraph:
    """Facade over the C-ABI graph handle; `generate_task_graph` is what demo.py:1179 calls directly."""

    def __init__(self, handle_owner):
        self._owner = handle_owner

    @property
    def handle(self):
        return self._owner._handle

    def generate_task_graph(self, num_gpus: int, my_gpu_id: int):
        json_text = self._owner._g.generate_task_graph(num_gpus, my_gpu_id)
        note = ("// The MI355X decode megakernel is precompiled (libfleet_mk.so) and data-driven:\n"
                "// no per-graph source is generated.  Stage program:\n")
        return {"json_file": json_text, "cuda_code": note + "// " + self._owner.describe_program().replace("\n", "\n// ")}

    def _torch_view(self, t):
        return self._owner._torch_view(t)
