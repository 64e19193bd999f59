"""`mirage`-compatible front end of the MI355X persistent decode megakernel.

Only the PersistentKernel (MPK) decode path of the reference package is provided:
`mi.PersistentKernel`, the dtype tags, `mi.get_configurations_from_gpu` and `mi.mpk.spec_decode_class`
(python/mirage/__init__.py, python/mirage/utils.py:38-101 in the reference).
"""
from .kernel import (DTensor, KNGraph, bfloat16, convert_dtype_to_torch_type, convert_torch_type_to_dtype, dtype, float16,
                     float32, int32, int64, uint64)
from . import mpk
from .mpk.persistent_kernel import PersistentKernel
from .mpk import speculative
from .utils import get_configurations_from_gpu

__all__ = ["PersistentKernel", "DTensor", "KNGraph", "dtype", "bfloat16", "float16", "float32", "int32", "int64", "uint64",
           "get_configurations_from_gpu", "mpk", "speculative", "convert_torch_type_to_dtype", "convert_dtype_to_torch_type"]
