"""PersistentKernel: the layer/task-builder API of the decode megakernel.

Same surface as the reference class (python/mirage/mpk/persistent_kernel.py:368-2786) for the
methods demo/qwen3/demo.py uses: each `*_layer` call validates shapes, then records one task
(name, grid, operands with their partition maps, params) through the C ABI.  `compile()` lowers the
recorded list to the MI355X stage program; `__call__` launches the persistent kernel once for the
whole generation.  Nothing here computes: without libfleet_mk.so and a gfx950 device it raises.
"""
import ctypes
import math
import os
import sys

import torch

from .. import _capi
from ..kernel import DTensor, KNGraph, bfloat16, convert_torch_type_to_dtype, int64

# the reference spells the multi-turn mode "online_multi_turn" (persistent_kernel.py:132); "multi_turn" is kept as an alias
valid_persistent_kernel_modes = ["offline", "online", "online_notoken", "onepass", "online_multi_turn", "multi_turn"]

_META_ORDER = ["step", "tokens", "input_tokens", "output_tokens", "num_new_tokens", "prompt_lengths",
               "qo_indptr_buffer", "paged_kv_indptr_buffer", "paged_kv_indices_buffer", "paged_kv_last_page_len_buffer"]

_REPL = (-1, -1, -1)


class PersistentKernel:
    def __init__(
        self,
        mode: str,
        world_size: int,
        mpi_rank: int,
        num_workers: int,
        num_local_schedulers: int,
        num_remote_schedulers: int,
        max_seq_length: int,
        max_num_batched_requests: int,
        max_num_batched_tokens: int,
        max_num_pages: int,
        page_size: int,
        meta_tensors: dict,
        profiler_tensor: torch.Tensor = None,
        trace_name: str = None,
        spec_decode_config=None,
        use_cutlass_kernel: bool = False,
        eos_token_id: int = -1,
        max_tokens_per_request: int = None,
        single_weight_copy: bool = None,
        binding: str = None,
    ):
        """Arguments as the reference constructor (persistent_kernel.py:368-387).  `max_tokens_per_request` is the
        reference's compile-time MPK_MAX_TOKENS_PER_REQUEST (prompt tokens one request ingests per iteration; 8 on AMD,
        persistent_kernel.cuh:115-124): None takes the environment variable of that name, else 8; at most 64.
        `single_weight_copy` (no counterpart in the reference; None takes FLEET_MK_SINGLE_WEIGHT_COPY, else False): a graph
        with max_num_batched_tokens >= 2 then keeps every linear weight ONCE, in the matrix-core tile layout compile()
        makes; `release_row_major_weights()` afterwards drops the attached tensors nothing reads any more.
        `binding`: "ctypes" or "cython" -- which binding of the C ABI carries the calls (None: FLEET_MK_BINDING, else ctypes)."""
        self.__finalized__ = False
        self._is_compiled = False
        self._handle = None
        if mode not in valid_persistent_kernel_modes:
            raise ValueError(f"Invalid persistent kernel mode: {mode}")
        if mode not in _capi.MK_MODES:
            raise NotImplementedError(f"mode '{mode}' is not supported by the MI355X megakernel (supported: {sorted(_capi.MK_MODES)})")
        if max_tokens_per_request is None:
            max_tokens_per_request = int(os.environ.get("MPK_MAX_TOKENS_PER_REQUEST", "8"))
        self.max_tokens_per_request = int(max_tokens_per_request)
        if world_size != 1 or mpi_rank != 0:
            raise NotImplementedError("the MI355X megakernel runs on one GPU (world_size=1, mpi_rank=0)")
        if spec_decode_config is not None:
            if getattr(spec_decode_config, "method", None) != "promptlookup":
                # (the reference registers handlers for prompt lookup only, persistent_kernel.py:410-415)
                raise NotImplementedError(f"speculative decoding method '{getattr(spec_decode_config, 'method', spec_decode_config)}' has no tasks; supported: promptlookup")
            if mode != "offline":
                raise NotImplementedError("speculative decoding needs mode 'offline': the on-GPU scheduler sizes the token groups of decoding requests")
            need = spec_decode_config.spec_length + 1
            if max_num_batched_tokens < need or self.max_tokens_per_request < need:
                raise ValueError(f"prompt lookup with {spec_decode_config.spec_length} guesses needs max_num_batched_tokens and max_tokens_per_request >= {need}")
        self.mode = mode
        self.world_size = world_size
        self.mpi_rank = mpi_rank
        self.num_workers = num_workers
        self.num_local_schedulers = num_local_schedulers
        self.num_remote_schedulers = num_remote_schedulers
        self.max_seq_length = max_seq_length
        self.max_num_batched_requests = max_num_batched_requests
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_num_pages = max_num_pages
        self.page_size = page_size
        self.eos_token_id = eos_token_id
        self.meta_tensors = meta_tensors
        self._profiler_tensor = profiler_tensor
        self._profiler_attached = False
        self.trace_name = trace_name
        self.use_nvshmem = False
        self.spec_decode_config = spec_decode_config
        self._spec_decode_handlers = {"promptlookup": self.prompt_lookup_spec_handler}
        self._spec_verify_handlers = {"promptlookup": self.prompt_lookup_verify_handler}
        self.use_cutlass_kernel = False
        self.is_rocm = True
        self.target_cc = 94  # the reference's tag for its MI300/MI350 task set (persistent_kernel.py:425-427)
        for key in _META_ORDER:
            if key not in meta_tensors:
                raise KeyError(f"meta_tensors is missing '{key}'")
        self.total_num_requests = meta_tensors["tokens"].shape[0]
        assert self.max_seq_length == meta_tensors["tokens"].shape[1]
        mt = meta_tensors
        assert mt["qo_indptr_buffer"].shape[0] <= max_num_batched_requests + 1, f"qo_indptr_buffer.shape: {mt['qo_indptr_buffer'].shape}"
        assert mt["paged_kv_indptr_buffer"].shape[0] <= max_num_batched_requests + 1, f"paged_kv_indptr_buffer.shape: {mt['paged_kv_indptr_buffer'].shape}"
        assert mt["paged_kv_indices_buffer"].shape[0] <= max_num_pages, f"paged_kv_indices_buffer.shape: {mt['paged_kv_indices_buffer'].shape}"
        assert mt["paged_kv_last_page_len_buffer"].shape[0] <= max_num_batched_requests, f"paged_kv_last_page_len_buffer.shape: {mt['paged_kv_last_page_len_buffer'].shape}"
        for key in ("tokens", "input_tokens", "output_tokens"):
            assert mt[key].dtype == torch.int64, f"{key}.dtype: {mt[key].dtype}"
        for key in ("step", "num_new_tokens", "prompt_lengths", "qo_indptr_buffer", "paged_kv_indptr_buffer",
                    "paged_kv_indices_buffer", "paged_kv_last_page_len_buffer"):
            assert mt[key].dtype == torch.int32, f"{key}.dtype: {mt[key].dtype}"
        # the library sizes the kernel-side buffers from the configuration, so the tensors must cover it
        assert mt["qo_indptr_buffer"].shape[0] == max_num_batched_requests + 1
        assert mt["paged_kv_indptr_buffer"].shape[0] == max_num_batched_requests + 1
        assert mt["paged_kv_indices_buffer"].shape[0] == max_num_pages
        assert mt["paged_kv_last_page_len_buffer"].shape[0] == max_num_batched_requests
        assert mt["input_tokens"].numel() >= max_num_batched_tokens and mt["output_tokens"].numel() >= max_num_batched_tokens
        device = mt["tokens"].device
        # CPU meta tensors give a host-only graph: layers can be recorded, validated, lowered and dumped as a task graph,
        # but compile() / __call__ raise -- the megakernel has no CPU path
        self.host_only = device.type != "cuda"
        self.device = device
        if single_weight_copy is None:
            single_weight_copy = os.environ.get("FLEET_MK_SINGLE_WEIGHT_COPY", "0") not in ("", "0")
        self.single_weight_copy = bool(single_weight_copy)
        cfg = dict(
            num_workers=int(num_workers) if num_workers else 0, max_seq_length=max_seq_length, max_num_batched_requests=max_num_batched_requests,
            max_num_batched_tokens=max_num_batched_tokens, max_num_pages=max_num_pages, page_size=page_size,
            total_num_requests=self.total_num_requests,
            device=-1 if self.host_only else (device.index if device.index is not None else torch.cuda.current_device()),
            eos_token_id=int(eos_token_id), rms_eps=1e-6, mode=_capi.MK_MODES[mode], max_tokens_per_request=self.max_tokens_per_request,
            flags=_capi.MK_CFG_SINGLE_WEIGHT_COPY if self.single_weight_copy else 0,
            step=mt["step"].data_ptr(), tokens=mt["tokens"].data_ptr(), input_tokens=mt["input_tokens"].data_ptr(),
            output_tokens=mt["output_tokens"].data_ptr(), num_new_tokens=mt["num_new_tokens"].data_ptr(),
            prompt_lengths=mt["prompt_lengths"].data_ptr(), qo_indptr=mt["qo_indptr_buffer"].data_ptr(),
            paged_kv_indptr=mt["paged_kv_indptr_buffer"].data_ptr(), paged_kv_indices=mt["paged_kv_indices_buffer"].data_ptr(),
            paged_kv_last_page_len=mt["paged_kv_last_page_len_buffer"].data_ptr())
        # the C ABI through the ctypes binding, or through the compiled Cython one (FLEET_MK_BINDING=cython / binding=)
        self._g = _capi.make_graph(cfg, binding)
        self._handle = ctypes.c_void_p(self._g.handle)  # for callers that talk to the C ABI directly
        self.kn_graph = KNGraph(self)
        self._tensors = []

    # ------------------------------------------------------------------ tensors
    def attach_input(self, torch_tensor: torch.Tensor, name: str = None) -> DTensor:
        dims = tuple(int(d) for d in torch_tensor.shape)
        strides = tuple(int(s) for s in torch_tensor.stride())
        for d in range(len(dims) - 1):
            assert strides[d] == strides[d + 1] * dims[d + 1], f"{name}: only row-major tensors can be attached"
        assert name is not None
        dt = convert_torch_type_to_dtype(torch_tensor.dtype)
        if (torch_tensor.device.type != "cuda") != self.host_only:
            raise RuntimeError(f"{name}: attached tensors must live on the same kind of device as the meta tensors")
        tid = self._g.tensor_attach(torch_tensor.data_ptr(), dims, strides, dt.code, name)
        t = DTensor(self, tid, dims, dt, name, torch_tensor)
        self._tensors.append(t)
        return t

    def new_tensor(self, dims: tuple, strides: tuple = None, dtype=bfloat16, name: str = None,
                   io_category: str = "cuda_tensor") -> DTensor:
        assert name is not None
        if io_category == "cuda_tensor":
            cat = 0
        elif io_category == "nvshmem_tensor":
            cat = 1
        else:
            raise RuntimeError(f"Invalid io_category: {io_category}")
        dims = tuple(int(d) for d in dims)
        tid = self._g.tensor_new(dims, None if strides is None else tuple(int(x) for x in strides), dtype.code, name, cat)
        t = DTensor(self, tid, dims, dtype, name)
        t._strides = tuple(strides) if strides is not None else None
        self._tensors.append(t)
        return t

    def _shuffle(self, inputs, dim, num_groups, name, interleave):
        ids = [t.id for t in inputs]
        tid = self._g.tensor_shuffle(ids, dim, num_groups, bool(interleave), name or "shuffled")
        rows = sum(t.dim(0) for t in inputs)
        t = DTensor(self, tid, (rows,) + tuple(inputs[0].shape[1:]), inputs[0].dtype, name)
        t.sources = list(inputs)
        self._tensors.append(t)
        return t

    def fuse_tensors(self, inputs: list, fused_dim: int, num_groups: int, name: str = None) -> DTensor:
        assert fused_dim == 0
        return self._shuffle(inputs, fused_dim, num_groups, name, True)

    def shuffle_tensors(self, inputs: list, shuffled_dim: int, num_groups: int, name: str = None) -> DTensor:
        assert shuffled_dim == 0
        return self._shuffle(inputs, shuffled_dim, num_groups, name, True)

    def _torch_view(self, t: DTensor):
        ptr = self._g.tensor_ptr(t.id)
        if not ptr:
            raise RuntimeError(f"tensor {t.name} has no device storage (shuffled views are resolved at run time)")
        n = 1
        strides = getattr(t, "_strides", None)
        if strides is None:
            for d in t.shape:
                n *= d
        else:
            n = 1 + sum((d - 1) * s for d, s in zip(t.shape, strides))
        holder = _DevicePtr(ptr, n * t.dtype.size, t.shape, t.dtype, self.device, strides)
        view = torch.as_tensor(holder, device=self.device)
        return view.view(torch.bfloat16) if t.dtype.name == "bfloat16" else view

    # ------------------------------------------------------------------ task recording
    def _task(self, name, grid_dim, block_dim, operands, params=()):
        """operands: list of (DTensor | None, input_map, forloop_dim), inputs first, outputs last."""
        assert not self._is_compiled, "graph already compiled"
        grid_dim = tuple(int(x) for x in grid_dim)
        block_dim = tuple(int(x) for x in block_dim)
        assert len(grid_dim) == 3 and len(block_dim) == 3
        ids, maps, fl = [], [], []
        for t, m, f in operands:
            ids.append(-1 if t is None else t.id)
            maps.extend(int(x) for x in m)
            fl.append(int(f))
        params = [int(p) for p in params]
        self._g.add_task(name, grid_dim, block_dim, ids, maps, fl, params)

    # ------------------------------------------------------------------ layers (reference line numbers in each docstring)
    def embed_layer(self, input: DTensor, weight: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple, input_source: int = 0):
        """persistent_kernel.py:521. input_source 0: ids are tokens[req, step+j]; 1: ids are the input tensor."""
        assert input.num_dims == 2 and weight.num_dims == 2 and output.num_dims == 2
        self._task("embedding", grid_dim, block_dim,
                   [(input, (-1, 1, -1), -1), (weight, (1, -1, -1), -1), (output, (1, 0, -1), -1)], [input_source])

    def rmsnorm_layer(self, input: DTensor, weight: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:544."""
        assert input.num_dims == 2 and weight.num_dims == 1 and output.num_dims == 2
        self._task("rmsnorm", grid_dim, block_dim,
                   [(input, (0, -1, -1), 1), (weight, _REPL, 0), (output, (0, -1, -1), 1)])

    def gang_rmsnorm_layer(self, input: DTensor, weight: DTensor, output: DTensor, block_dim: tuple = (128, 1, 1)):
        """persistent_kernel.py:1553."""
        assert input.num_dims == 2 and weight.num_dims == 1 and output.num_dims == 2
        self._task("gang_rmsnorm_mi300", (8, 1, 1), block_dim,
                   [(input, _REPL, -1), (weight, _REPL, -1), (output, _REPL, -1)], [input.dim(0)])

    def linear_layer(self, input: DTensor, weight: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2045."""
        assert input.num_dims == 2 and weight.num_dims == 2 and output.num_dims == 2
        self._task("linear", grid_dim, block_dim,
                   [(input, _REPL, 1), (weight, (0, -1, -1), 1), (output, (1, -1, -1), -1)])

    def linear_with_residual_layer(self, input: DTensor, weight: DTensor, residual: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2077."""
        assert input.num_dims == 2 and weight.num_dims == 2 and residual.num_dims == 2 and output.num_dims == 2
        self._task("linear_with_residual", grid_dim, block_dim,
                   [(input, _REPL, 1), (weight, (0, -1, -1), 1), (residual, (1, -1, -1), -1), (output, (1, -1, -1), -1)])

    def splitk_linear_res_atomic_layer(self, input: DTensor, weight: DTensor, residual: DTensor, workspace: DTensor, done_counter: DTensor,
                                       output: DTensor, k_splits: int, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:1920.  The MI355X kernel needs no split-K workspace; the operands are accepted and unused."""
        assert input.num_dims == 2 and weight.num_dims == 2 and residual.num_dims == 2 and output.num_dims == 2
        assert grid_dim[1] == k_splits
        assert input.dim(1) % k_splits == 0
        self._task("splitk_linear_res_atomic_mi300", grid_dim, block_dim,
                   [(input, (-1, 1, -1), 1), (weight, (0, 1, -1), 1), (residual, (1, -1, -1), -1), (workspace, (1, -1, -1), -1),
                    (done_counter, (0, -1, -1), -1), (output, (1, -1, -1), -1)], [k_splits])

    def splitk_linear_layer(self, input: DTensor, weight: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:1437.  grid_dim = (N blocks, K splits, 1).  With a bf16 [tokens, N] output it is lowered
        like linear_layer (the stage decides by itself whether to split K over workgroups, and sums the slices in a fixed
        order); with the reference's fp32 [k_splits * tokens, N] workspace as output it must be followed by
        splitk_reduce_layer over that workspace, and the pair becomes one linear stage."""
        assert input.num_dims == 2 and weight.num_dims == 2 and output.num_dims == 2
        self._task("splitk_linear_mi300", grid_dim, block_dim,
                   [(input, (-1, 1, -1), 1), (weight, (0, 1, -1), 1), (output, (1, 0, -1), -1)])

    def splitk_reduce_layer(self, workspace: DTensor, residual: DTensor, output: DTensor, k_splits: int, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:1901: output = bf16(sum of the k_splits slices of `workspace` + residual).  Closes a
        splitk_linear_layer whose output is that workspace; no partial sums are ever written to it."""
        assert workspace.num_dims == 2  # (k_splits * batch_size, hidden_size)
        assert residual.num_dims == 2   # (batch_size, hidden_size)
        assert output.num_dims == 2     # (batch_size, hidden_size)
        self._task("splitk_reduce_mi300", grid_dim, block_dim,
                   [(workspace, (1, -1, -1), 1), (residual, (1, -1, -1), 1), (output, (1, -1, -1), -1)], [k_splits])

    def silu_mul_linear_with_residual_layer(self, input: DTensor, weight: DTensor, residual: DTensor, output: DTensor, grid_dim: tuple,
                                            block_dim: tuple, gate_rows_per_group: int = None):
        """persistent_kernel.py:2174: output = bf16(silu_mul(input) @ weight^T + residual) with input = the gate/up linear's
        [tokens, 2 * intermediate] result.  Which columns are gate and which are up: the shuffled weight view of the linear
        that produced `input` says so; a caller that interleaved a physical weight itself passes `gate_rows_per_group`
        (not a reference argument: groups of [gate x n ; up x n]); otherwise `input` is read as [gate | up] halves, the
        layout the reference task kernel reads (tasks/mi300/silu_mul_linear_mi300.cuh:40-42).  The activation is folded into
        the producing linear's epilogue when nothing else reads `input`."""
        assert input.num_dims == 2  # (batch_size, 2*intermediate_size)
        assert weight.num_dims == 2  # (hidden_size, intermediate_size)
        assert residual.num_dims == 2  # (batch_size, hidden_size)
        assert input.dim(1) == 2 * weight.dim(1)
        self._task("silu_mul_linear_with_residual", grid_dim, block_dim,
                   [(input, _REPL, 1), (weight, (0, -1, -1), 1), (residual, (1, -1, -1), 1), (output, (1, -1, -1), 1)],
                   [int(gate_rows_per_group)] if gate_rows_per_group else [])

    # ------------------------------------------------------------------ mixture-of-experts layers
    def moe_topk_softmax_routing_layer(self, input: DTensor, output: tuple, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:1203.  fp32 softmax over all experts -> top-k (ties to the lower expert id) -> renormalise.
        Unlike the reference task (moe_topk_softmax_mi300.cuh:116-122) the router logits are left intact."""
        assert input.num_dims == 2  # (batch_size, num_experts)
        assert len(output) == 3
        moe_topk_weight, moe_routing_indices, moe_masks = output
        assert moe_topk_weight.num_dims == 2  # (batch_size, num_experts_per_tok)
        assert moe_routing_indices.num_dims == 2  # (num_experts, batch_size)
        assert moe_masks.num_dims == 1  # (num_experts + 1)
        self._task("moe_topk_softmax_mi300", grid_dim, block_dim,
                   [(input, (0, -1, -1), -1), (moe_topk_weight, (0, -1, -1), -1), (moe_routing_indices, _REPL, -1), (moe_masks, _REPL, -1)])

    def _moe_linear(self, name, input, weight, moe_routing_indices, moe_mask, output, grid_dim, block_dim, in_forloop, params=()):
        assert weight.num_dims == 3  # (num_experts, output_size, reduction_size)
        assert moe_routing_indices.num_dims == 2  # (num_experts, batch_size)
        assert moe_mask.num_dims == 1  # (num_experts + 1)
        assert output.num_dims == 3  # (batch_size, num_experts_per_tok, output_size)
        self._task(name, grid_dim, block_dim,
                   [(input, _REPL, in_forloop), (weight, (-1, 1, -1), 2), (moe_routing_indices, _REPL, -1), (moe_mask, _REPL, -1),
                    (output, (-1, 2, -1), -1)], params)

    def moe_w13_linear_layer(self, input: DTensor, weight: DTensor, moe_routing_indices: DTensor, moe_mask: DTensor, output: DTensor,
                             grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:1229.  output[t, slot, :] = weight[expert(t, slot)] @ input[t]."""
        assert input.num_dims == 2  # (batch_size, hidden_size)
        self._moe_linear("moe_w13_linear_mi300", input, weight, moe_routing_indices, moe_mask, output, grid_dim, block_dim, 1)

    def moe_silu_mul_layer(self, input: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:1262.  Rows are [gate ; up] halves per (token, slot)."""
        assert input.num_dims == 3  # (batch_size, num_experts_per_tok, 2 * intermediate_size)
        assert output.num_dims == 3  # (batch_size, num_experts_per_tok, intermediate_size)
        self._task("moe_silu_mul", grid_dim, block_dim, [(input, (0, 1, -1), -1), (output, (0, 1, -1), -1)])

    def moe_w2_linear_layer(self, input: DTensor, weight: DTensor, moe_routing_indices: DTensor, moe_mask: DTensor, output: DTensor,
                            grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:1278.  output[t, slot, :] = weight[expert(t, slot)] @ input[t, slot]."""
        assert input.num_dims == 3  # (batch_size, num_experts_per_tok, intermediate_size)
        self._moe_linear("moe_w2_linear_mi300", input, weight, moe_routing_indices, moe_mask, output, grid_dim, block_dim, 2)

    def _gang_moe_params(self, weight, k_multiple, per_token):
        batch_size = self.max_num_batched_tokens
        num_experts, output_size, reduction_size = weight.dim(0), weight.dim(1), weight.dim(2)
        tile_n = 64
        assert output_size % tile_n == 0, f"output_size {output_size} not divisible by {tile_n}"
        assert reduction_size % k_multiple == 0, f"K={reduction_size} not divisible by {k_multiple}"
        n_tiles = output_size // tile_n
        tiles_per_expert = n_tiles * batch_size if per_token else max(1, batch_size // 16) * n_tiles
        max_experts_per_xcd = (num_experts + 7) // 8
        total_tiles_per_xcd = max_experts_per_xcd * tiles_per_expert
        assert total_tiles_per_xcd <= 65535, f"total_tiles_per_xcd={total_tiles_per_xcd} exceeds uint16_t (bs={batch_size})"
        return [tiles_per_expert, max_experts_per_xcd, total_tiles_per_xcd]

    def gang_moe_w13_linear_layer(self, input: DTensor, weight: DTensor, moe_routing_indices: DTensor, moe_mask: DTensor, output: DTensor,
                                  block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1311.  Same stage as moe_w13_linear_layer."""
        assert input.num_dims == 2
        self._moe_linear("gang_moe_w13_linear_mi300", input, weight, moe_routing_indices, moe_mask, output, (8, 1, 1), block_dim, 1,
                         self._gang_moe_params(weight, 256, False))

    def gang_moe_w2_linear_layer(self, input: DTensor, weight: DTensor, moe_routing_indices: DTensor, moe_mask: DTensor, output: DTensor,
                                 block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1361.  Same stage as moe_w2_linear_layer."""
        assert input.num_dims == 3
        self._moe_linear("gang_moe_w2_linear_mi300", input, weight, moe_routing_indices, moe_mask, output, (8, 1, 1), block_dim, 2,
                         self._gang_moe_params(weight, 128, True))

    def moe_mul_sum_add_layer(self, input: DTensor, weight: DTensor, residual: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:1411.  output = residual + sum_k weight[t, k] * input[t, k, :] in fp32."""
        assert input.num_dims == 3  # (batch_size, num_experts_per_tok, hidden_size)
        assert weight.num_dims == 2  # (batch_size, num_experts_per_tok)
        assert residual.num_dims == 2 and output.num_dims == 2
        self._task("moe_mul_sum_add_mi300", grid_dim, block_dim,
                   [(input, (0, 2, -1), -1), (weight, (0, -1, -1), -1), (residual, (0, 1, -1), -1), (output, (0, 1, -1), -1)])

    def _gang_params(self, weight, tile_n, output_stride, m_tiles, wg, out_rows=None):
        batch_size = self.max_num_batched_tokens
        output_size = weight.dim(0) if out_rows is None else out_rows
        assert output_size % 8 == 0, f"Output size {output_size} must be divisible by 8"
        chunk_n = output_size // 8
        assert chunk_n % tile_n == 0, f"Chunk {chunk_n} must be divisible by tile_n {tile_n}"
        n_tiles_per_xcd = chunk_n // tile_n
        assert batch_size % m_tiles == 0, f"batch {batch_size} must be divisible by m_tiles {m_tiles}"
        m_per_tile = batch_size // m_tiles
        return [output_stride, tile_n, m_tiles, m_per_tile, n_tiles_per_xcd * m_tiles, n_tiles_per_xcd, wg]

    def gang_linear_layer(self, input: DTensor, weight: DTensor, output: DTensor, tile_n: int, output_stride: int, m_tiles: int = 1,
                          wgm: int = 0, block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1571."""
        assert input.num_dims == 2 and weight.num_dims == 2 and output.num_dims == 2
        self._task("gang_linear_mi300", (8, 1, 1), block_dim,
                   [(input, _REPL, 1), (weight, (0, -1, -1), 1), (output, (1, -1, -1), -1)],
                   self._gang_params(weight, tile_n, output_stride, m_tiles, wgm))

    def gang_linear_n_tiling_layer(self, input: DTensor, weight: DTensor, output: DTensor, tile_n: int, output_stride: int, m_tiles: int = 1,
                                   wgn: int = 0, block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1618 (tile traversal variant; same mathematics)."""
        assert input.num_dims == 2 and weight.num_dims == 2 and output.num_dims == 2
        self._task("gang_linear_n_tiling_mi300", (8, 1, 1), block_dim,
                   [(input, _REPL, 1), (weight, (0, -1, -1), 1), (output, (1, -1, -1), -1)],
                   self._gang_params(weight, tile_n, output_stride, m_tiles, wgn))

    def gang_linear_with_residual_layer(self, input: DTensor, weight: DTensor, residual: DTensor, output: DTensor, tile_n: int,
                                        output_stride: int, m_tiles: int = 1, wgm: int = 0, block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1670."""
        assert input.num_dims == 2 and weight.num_dims == 2 and residual.num_dims == 2 and output.num_dims == 2
        self._task("gang_linear_res_mi300", (8, 1, 1), block_dim,
                   [(input, _REPL, 1), (weight, (0, -1, -1), 1), (residual, (1, -1, -1), -1), (output, (1, -1, -1), -1)],
                   self._gang_params(weight, tile_n, output_stride, m_tiles, wgm))

    def gang_linear_with_residual_n_tiling_layer(self, input: DTensor, weight: DTensor, residual: DTensor, output: DTensor, tile_n: int,
                                                 output_stride: int, m_tiles: int = 1, wgn: int = 0, block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1737."""
        assert input.num_dims == 2 and weight.num_dims == 2 and residual.num_dims == 2 and output.num_dims == 2
        self._task("gang_linear_res_n_tiling_mi300", (8, 1, 1), block_dim,
                   [(input, _REPL, 1), (weight, (0, -1, -1), 1), (residual, (1, -1, -1), -1), (output, (1, -1, -1), -1)],
                   self._gang_params(weight, tile_n, output_stride, m_tiles, wgn))

    def _msplit_params(self, weight, tile_n, output_stride, m_tiles):
        batch_size = self.max_num_batched_tokens
        output_size = weight.dim(0)
        assert output_size % 8 == 0 and (output_size // 8) % tile_n == 0
        assert batch_size % m_tiles == 0
        n_tiles_per_xcd = output_size // 8 // tile_n
        return [output_stride, tile_n, m_tiles, n_tiles_per_xcd, batch_size // m_tiles]

    def gang_linear_msplit_layer(self, input: DTensor, weight: DTensor, output: DTensor, tile_n: int, output_stride: int, m_tiles: int = 2,
                                 block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1782."""
        assert input.num_dims == 2 and weight.num_dims == 2 and output.num_dims == 2
        self._task("gang_linear_msplit_mi300", (8 * m_tiles, 1, 1), block_dim,
                   [(input, _REPL, 1), (weight, _REPL, 1), (output, _REPL, -1)], self._msplit_params(weight, tile_n, output_stride, m_tiles))

    def gang_linear_with_residual_msplit_layer(self, input: DTensor, weight: DTensor, residual: DTensor, output: DTensor, tile_n: int,
                                               output_stride: int, m_tiles: int = 2, block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1817."""
        assert input.num_dims == 2 and weight.num_dims == 2 and residual.num_dims == 2 and output.num_dims == 2
        self._task("gang_linear_res_msplit_mi300", (8 * m_tiles, 1, 1), block_dim,
                   [(input, _REPL, 1), (weight, _REPL, 1), (residual, _REPL, -1), (output, _REPL, -1)],
                   self._msplit_params(weight, tile_n, output_stride, m_tiles))

    def gang_splitk_linear_with_residual_layer(self, input: DTensor, weight: DTensor, residual: DTensor, workspace: DTensor, output: DTensor,
                                               tile_n: int, output_stride: int, k_splits: int = 4, block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1515.  Computed without split-K atomics (deterministic); the workspace is unused."""
        assert input.num_dims == 2 and weight.num_dims == 2 and residual.num_dims == 2 and output.num_dims == 2
        output_size = weight.dim(0)
        assert output_size % 8 == 0 and (output_size // 8) % tile_n == 0
        self._task("gang_splitk_linear_res_mi300", (8, 1, 1), block_dim,
                   [(input, _REPL, 1), (weight, (0, -1, -1), 1), (residual, (1, -1, -1), -1), (workspace, (1, -1, -1), -1), (output, (1, -1, -1), -1)],
                   [output_stride, tile_n, output_size // 8 // tile_n, k_splits])

    def gang_ksplit_linear_with_residual_layer(self, input, weight, residual, workspace, output, tile_n, output_stride, k_splits=8,
                                               block_dim=(256, 1, 1)):
        """persistent_kernel.py:1468.  Same mathematics as gang_linear_with_residual_layer; lowered identically."""
        return self.gang_splitk_linear_with_residual_layer(input, weight, residual, workspace, output, tile_n, output_stride, k_splits, block_dim)

    def gang_linear_silu_layer(self, input: DTensor, weight: DTensor, output: DTensor, tile_n: int, output_stride: int, m_tiles: int = 1,
                               wgm: int = 0, block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1852.  weight interleaves [gate ; up] groups; output has half as many columns."""
        assert input.num_dims == 2 and weight.num_dims == 2 and output.num_dims == 2
        assert weight.dim(0) % 2 == 0 and output.dim(1) * 2 == weight.dim(0), "output must have weight.dim(0)/2 columns"
        self._task("gang_linear_silu_mi300", (8, 1, 1), block_dim,
                   [(input, _REPL, 1), (weight, (0, -1, -1), 1), (output, (1, -1, -1), -1)],
                   self._gang_params(weight, tile_n, output_stride, m_tiles, wgm, out_rows=weight.dim(0) // 2))

    def linear_silu_layer(self, input, weight, output, output_stride, tile_n=64, m_tiles=1, wgm=0, block_dim=(256, 1, 1)):
        """persistent_kernel.py:1716."""
        assert input.num_dims == 2 and weight.num_dims == 2 and output.num_dims == 2
        assert weight.dim(0) % 2 == 0 and output.dim(1) * 2 == weight.dim(0), "output must have weight.dim(0)/2 columns"
        batch_size = self.max_num_batched_tokens
        n_output_tiles = weight.dim(0) // tile_n // 2
        m_per_tile = batch_size // m_tiles if m_tiles > 0 else batch_size
        total_tiles = n_output_tiles * m_tiles
        self._task("linear_silu_mi300", (total_tiles, 1, 1), block_dim,
                   [(input, _REPL, 1), (weight, _REPL, 1), (output, _REPL, -1)],
                   [output_stride, tile_n, m_tiles, m_per_tile, total_tiles, n_output_tiles, wgm])

    def silu_mul_layer(self, input: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2137.  Each of the grid_dim[0] blocks owns one [gate ; up] column group."""
        assert input.num_dims == 2 and output.num_dims == 2
        assert input.dim(1) == 2 * output.dim(1)
        self._task("silu_mul", grid_dim, block_dim, [(input, (1, -1, -1), -1), (output, (1, -1, -1), -1)])

    def kv_cache_update_layer(self, input: DTensor, k_cache: DTensor, v_cache: DTensor, q_norm: DTensor, k_norm: DTensor,
                              cos_pos_embed: DTensor, sin_pos_embed: DTensor, q_workspace: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:937."""
        assert input.num_dims == 2
        assert k_cache.num_dims == 4 and v_cache.num_dims == 4
        assert q_workspace.num_dims == 2
        head_dim = k_cache.dim(3)
        num_kv_heads = k_cache.dim(2)
        num_q_heads = q_workspace.dim(1) // head_dim
        rotary_embed = 1 if cos_pos_embed is not None else 0
        qk_norm = 1 if q_norm is not None else 0
        params = [num_q_heads, num_kv_heads, qk_norm, rotary_embed, self.max_seq_length, self.page_size, q_workspace.dim(1)]
        self._task("kv_cache_update_mi300", grid_dim, block_dim,
                   [(input, (-1, 1, -1), -1), (k_cache, (-1, 2, -1), 1), (v_cache, (-1, 2, -1), 1), (q_norm, _REPL, -1), (k_norm, _REPL, -1),
                    (cos_pos_embed, _REPL, -1), (sin_pos_embed, _REPL, -1), (q_workspace, (-1, 1, -1), -1)], params)

    def paged_attention_ck_fmha_layer(self, q_workspace: DTensor, k_cache: DTensor, v_cache: DTensor, o_acc: DTensor, lse_acc: DTensor,
                                      attention_params: tuple, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:981.  With num_kv_chunks == 1 `o_acc` is the final bf16 attention output; with more chunks it is
        the reference's fp32 accumulator and paged_attention_ck_fmha_merge_layer must follow."""
        assert q_workspace.num_dims == 2
        assert k_cache.num_dims == 4 and v_cache.num_dims == 4
        assert o_acc.num_dims == 2 and lse_acc.num_dims == 2
        head_dim = k_cache.dim(3)
        num_kv_heads = k_cache.dim(2)
        num_q_heads, num_kv_chunks, num_requests = attention_params[0], attention_params[1], attention_params[2]
        kv_stride = num_kv_heads * head_dim
        params = [num_q_heads, num_kv_heads, head_dim, self.page_size, self.max_seq_length, num_kv_chunks, q_workspace.dim(1), kv_stride, num_requests]
        self._task("paged_attention_ck_fmha_split_kv_mi300", grid_dim, block_dim,
                   [(q_workspace, _REPL, -1), (k_cache, (-1, 2, -1), 1), (v_cache, (-1, 2, -1), 1), (o_acc, _REPL, -1), (lse_acc, _REPL, -1)], params)

    def gang_paged_attention_split_kv_layer(self, input: DTensor, k_cache: DTensor, v_cache: DTensor, q_norm: DTensor, k_norm: DTensor,
                                            cos_pos_embed: DTensor, sin_pos_embed: DTensor, lse: DTensor, output: DTensor, q_workspace: DTensor,
                                            attention_params: tuple, block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1064: KV append + q/k-norm + RoPE + attention in one task."""
        assert input.num_dims == 2
        assert k_cache.num_dims == 4 and v_cache.num_dims == 4
        num_kv_heads = k_cache.dim(2)
        num_q_heads, num_kv_chunks, q_workspace_stride = attention_params[0], attention_params[1], attention_params[2]
        rotary_embed = 0
        if cos_pos_embed is not None or sin_pos_embed is not None:
            assert cos_pos_embed.num_dims == 2 and sin_pos_embed.num_dims == 2
            rotary_embed = 1
        qk_norm = 0
        if q_norm is not None or k_norm is not None:
            assert q_norm.num_dims == 1 and k_norm.num_dims == 1
            qk_norm = 1
        total = self.max_num_batched_requests * num_kv_heads * num_kv_chunks
        params = [num_q_heads, num_kv_heads, qk_norm, rotary_embed, self.max_seq_length, self.page_size, num_kv_chunks,
                  math.ceil(total / 8), total, q_workspace_stride]
        self._task("gang_attn_split_kv_mi300", (8, 1, 1), block_dim,
                   [(input, _REPL, 1), (k_cache, _REPL, 1), (v_cache, _REPL, 1), (q_norm, _REPL, -1), (k_norm, _REPL, -1), (cos_pos_embed, _REPL, -1),
                    (sin_pos_embed, _REPL, -1), (lse, _REPL, -1), (output, _REPL, -1), (q_workspace, _REPL, -1)], params)

    def argmax_partial_layer(self, input: DTensor, output: tuple, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2207."""
        assert input.num_dims == 2
        assert len(output) == 2
        output_value, output_index = output
        assert output_value.num_dims == 2 and output_index.num_dims == 2
        num_tasks = grid_dim[0]
        self.argmax_partial_output_size = input.dim(1) // num_tasks
        self._task("argmax_partial", grid_dim, block_dim,
                   [(input, (1, 0, -1), -1), (output_value, (1, 0, -1), -1), (output_index, (1, 0, -1), -1)], [num_tasks])

    def argmax_reduce_layer(self, input: tuple, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2232."""
        assert len(input) == 2
        input_value, input_index = input
        assert input_value.num_dims == 2 and input_index.num_dims == 2
        assert output.num_dims == 2
        self._task("argmax_reduce", grid_dim, block_dim,
                   [(input_value, (1, 0, -1), -1), (input_index, (1, 0, -1), -1), (output, (0, 1, -1), -1)],
                   [getattr(self, "argmax_partial_output_size", 0)])

    def rmsnorm_linear_layer(self, input: DTensor, weight_norm: DTensor, weight_linear: DTensor, output: DTensor, grid_dim: tuple,
                             block_dim: tuple):
        """persistent_kernel.py:566: output = linear(rmsnorm(input, weight_norm), weight_linear) as one task.  Lowered as
        the norm + linear pair (a single-token iteration computes the norm inside the linear stage)."""
        assert input.num_dims == 2
        assert weight_linear.num_dims == 2
        assert output.num_dims == 2
        self._task("rmsnorm_linear", grid_dim, block_dim,
                   [(input, _REPL, 1), (weight_norm, _REPL, 0), (weight_linear, (0, -1, -1), 1), (output, (1, -1, -1), -1)])

    def attention_layer(self, input: DTensor, k_cache: DTensor, v_cache: DTensor, q_norm: DTensor, k_norm: DTensor, cos_pos_embed: DTensor,
                        sin_pos_embed: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:587: the form whose caches are [requests, seq_len, kv_heads, head_dim], one contiguous
        range of rows per request -- a paged cache with pages of max_seq_length rows, so the graph must be built with
        page_size == seq_len and at least one page per request.  Same stage as every other attention builder."""
        assert input.num_dims == 2  # (batch_size, fused_outdim)
        assert output.num_dims == 2  # (batch_size, hidden_size)
        assert k_cache.num_dims == 4 and v_cache.num_dims == 4  # (batch_size, seq_len, kv_heads, head_dim)
        head_dim, num_kv_heads = k_cache.dim(3), k_cache.dim(2)
        num_q_heads = output.dim(1) // head_dim
        qk_norm, rotary_embed = self._attn_flags(q_norm, k_norm, cos_pos_embed, sin_pos_embed, head_dim)
        assert k_cache.dim(1) == self.page_size, "attention_layer: one page per request (page_size == the cache's seq_len)"
        self._task("attention", grid_dim, block_dim,
                   [(input, (0, 1, -1), -1), (k_cache, (0, 2, -1), 1), (v_cache, (0, 2, -1), 1), (q_norm, _REPL, -1), (k_norm, _REPL, -1),
                    (cos_pos_embed, _REPL, -1), (sin_pos_embed, _REPL, -1), (output, (0, 1, -1), -1)],
                   [num_q_heads, num_kv_heads, qk_norm, rotary_embed])

    def identity_layer(self, input: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple, dependent_tensor: DTensor = None):
        """persistent_kernel.py:2153: output = input (the rows of the running iteration)."""
        last_dim = 0
        assert input.num_dims == output.num_dims
        for i in range(input.num_dims):
            assert input.dim(i) == output.dim(i)
            last_dim = i
        assert last_dim == 1 or last_dim == 2
        self._task("identity", grid_dim, block_dim, [(input, (last_dim, -1, -1), 1), (output, (last_dim, -1, -1), 1)])

    def argmax_layer(self, input: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2195: greedy token of every row in one task (lowest index on ties)."""
        assert input.num_dims == 2  # (batch_size, vocab_size)
        assert output.num_dims == 2  # (batch_size, 1)
        self._task("argmax", grid_dim, block_dim, [(input, _REPL, -1), (output, _REPL, -1)])

    def linear_m_parallel_layer(self, input: DTensor, weight: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:1953: the plain linear task with grid (N tiles, M tiles, 1)."""
        assert input.num_dims == 2 and weight.num_dims == 2 and output.num_dims == 2
        self._task("linear", grid_dim, block_dim, [(input, (-1, 0, -1), 1), (weight, (0, -1, -1), 1), (output, (1, 0, -1), -1)])

    def linear_with_residual_m_parallel_layer(self, input: DTensor, weight: DTensor, residual: DTensor, output: DTensor, grid_dim: tuple,
                                              block_dim: tuple):
        """persistent_kernel.py:1977."""
        assert input.num_dims == 2 and weight.num_dims == 2 and residual.num_dims == 2 and output.num_dims == 2
        self._task("linear_with_residual", grid_dim, block_dim,
                   [(input, (-1, 0, -1), 1), (weight, (0, -1, -1), 1), (residual, (1, 0, -1), 1), (output, (1, 0, -1), -1)])

    def splitk_linear_res_atomic_m_parallel_layer(self, input: DTensor, weight: DTensor, residual: DTensor, workspace: DTensor,
                                                  done_counter: DTensor, output: DTensor, k_splits: int, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2002: grid (N tiles, K splits, M tiles); the sum is deterministic here and the workspace and
        counters stay untouched."""
        assert input.num_dims == 2 and weight.num_dims == 2
        self._task("splitk_linear_res_atomic_mi300", grid_dim, block_dim,
                   [(input, (-1, 1, 0), 1), (weight, (0, 1, -1), 1), (residual, (1, -1, 0), 1), (workspace, (1, -1, 0), 1),
                    (done_counter, (0, -1, 1), 1), (output, (1, -1, 0), -1)], [k_splits])

    # layers of the reference that are outside the one-GPU decode path
    def tensor_init_layer(self, *args, **kwargs):
        raise NotImplementedError("tensor_init_layer registers a Blackwell-only task (tasks/blackwell/tensor_init.cuh); it has no MI300-family kernel in the reference either")

    def allreduce_layer(self, *args, **kwargs):
        raise NotImplementedError("allreduce_layer: the MI355X megakernel runs on one GPU")

    # ------------------------------------------------------------------ prompt-lookup speculative decoding
    def find_ngram_partial_layer(self, input: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple, ngram_size: int = 3):
        """persistent_kernel.py:2279.  input = the `tokens` meta tensor; output[slot, task] = the earliest position in the
        task's share of the request's history where its last `ngram_size` tokens occurred before (int64 max: nowhere)."""
        assert input.num_dims == 2  # (requests, seq_len)
        assert output.num_dims == 2  # (batch slots, num_tasks)
        self._task("find_ngram_partial", grid_dim, block_dim, [(input, _REPL, -1), (output, (1, -1, -1), -1)], [ngram_size])

    def find_ngram_global_layer(self, input: tuple, output: DTensor, grid_dim: tuple, block_dim: tuple, ngram_size: int = 3, spec_length: int = 5):
        """persistent_kernel.py:2290.  output = the token ids of the iteration's rows: the scheduler's, and behind a decoding
        request's newest token the `spec_length` tokens that followed the earliest match (-1 where there are none)."""
        assert len(input) == 2
        partial_results, tokens = input
        assert partial_results.num_dims == 2  # (batch slots, num_tasks)
        assert tokens.num_dims == 2
        assert output.num_dims == 2
        self._task("find_ngram_global", grid_dim, block_dim, [(partial_results, _REPL, -1), (tokens, _REPL, -1), (output, _REPL, -1)],
                   [ngram_size, spec_length])

    def prompt_lookup_spec_handler(self, spec_decode_config, tokens: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2305: the two n-gram tasks; returns the tensor the embedding layer reads its ids from.
        Sized for every token row of an iteration (the reference sizes it for its single request: [1, spec_length + 1])."""
        slots = max(tokens.dim(0), self.max_num_batched_requests)
        partial_ngram_output = self.new_tensor(dims=(slots, 96), dtype=int64, name="partial_ngram_output", io_category="cuda_tensor")
        self.find_ngram_partial_layer(input=tokens, output=partial_ngram_output, grid_dim=grid_dim, block_dim=block_dim,
                                      ngram_size=spec_decode_config.ngram_size)
        width = spec_decode_config.spec_length + 1
        rows = max(tokens.dim(0), -(-self.max_num_batched_tokens // width))  # one id per token row of an iteration, row-major
        spec_tokens = self.new_tensor(dims=(rows, width), dtype=int64, name="spec_tokens", io_category="cuda_tensor")
        self.find_ngram_global_layer(input=(partial_ngram_output, tokens), output=spec_tokens, grid_dim=(1, 1, 1), block_dim=(128, 1, 1),
                                     ngram_size=spec_decode_config.ngram_size, spec_length=spec_decode_config.spec_length)
        return spec_tokens

    def draft_forward_layer_dispatcher(self, spec_decode_config, tokens: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2341."""
        handler = self._spec_decode_handlers.get(spec_decode_config.method)
        if handler is None:
            raise ValueError(f"Invalid spec decode method: {spec_decode_config.method}")
        return handler(spec_decode_config, tokens, grid_dim, block_dim)

    def target_verify_greedy_layer(self, input: tuple, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2354.  Counts, per decoding request, the sampled tokens it keeps (1 + the leading guesses the
        model agreed with) into the num_new_tokens meta tensor; `output` receives batch slot 0's count."""
        assert len(input) == 2
        spec_tokens, target_tokens = input
        assert spec_tokens.num_dims == 2 and target_tokens.num_dims == 2 and output.num_dims == 2
        self._task("target_verify_greedy", grid_dim, block_dim, [(spec_tokens, _REPL, -1), (target_tokens, _REPL, -1), (output, _REPL, -1)])

    def prompt_lookup_verify_handler(self, spec_decode_config, spec_tokens: DTensor, target_output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:2370."""
        verify_out = self.new_tensor(dims=(1, 1), dtype=int64, name="verify_out", io_category="cuda_tensor")
        self.target_verify_greedy_layer(input=(spec_tokens, target_output), output=verify_out, grid_dim=grid_dim, block_dim=block_dim)
        return verify_out

    def verify_layer_dispatcher(self, spec_decode_config, spec_tokens: DTensor, target_output: DTensor, grid_dim: tuple = (1, 1, 1),
                                block_dim: tuple = (128, 1, 1)):
        """persistent_kernel.py:2389."""
        handler = self._spec_verify_handlers.get(spec_decode_config.method)
        if handler is None:
            raise ValueError(f"Invalid spec decode method: {spec_decode_config.method}")
        return handler(spec_decode_config, spec_tokens, target_output, grid_dim, block_dim)

    def single_batch_extend_attention_layer(self, input: DTensor, k_cache: DTensor, v_cache: DTensor, q_norm: DTensor, k_norm: DTensor,
                                            cos_pos_embed: DTensor, sin_pos_embed: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:653: attention over the rows of a speculating request (its newest token and the guesses
        behind it, causal among themselves), caches [requests, seq_len, kv_heads, head_dim].  The attention stage handles
        several new rows of one request in any case, so this lowers like attention_layer."""
        assert input.num_dims == 2 and output.num_dims == 2
        assert k_cache.num_dims == 4 and v_cache.num_dims == 4
        head_dim, num_kv_heads = k_cache.dim(3), k_cache.dim(2)
        num_q_heads = output.dim(1) // head_dim
        qk_norm, rotary_embed = self._attn_flags(q_norm, k_norm, cos_pos_embed, sin_pos_embed, head_dim)
        assert k_cache.dim(1) == self.page_size, "single_batch_extend_attention_layer: one page per request (page_size == the cache's seq_len)"
        self._task("single_batch_extend_attention", grid_dim, block_dim,
                   [(input, (0, 1, -1), -1), (k_cache, (0, 2, -1), 1), (v_cache, (0, 2, -1), 1), (q_norm, _REPL, -1), (k_norm, _REPL, -1),
                    (cos_pos_embed, _REPL, -1), (sin_pos_embed, _REPL, -1), (output, (0, 1, -1), -1)],
                   [num_q_heads, num_kv_heads, qk_norm, rotary_embed, input.dim(0) - 1, output.dim(1)])

    # ------------------------------------------------------------------ attention variants that lower to the same stage
    def _attn_flags(self, q_norm, k_norm, cos_pos_embed, sin_pos_embed, head_dim):
        rotary_embed = 0
        if cos_pos_embed is not None or sin_pos_embed is not None:
            assert cos_pos_embed.num_dims == 2 and sin_pos_embed.num_dims == 2  # (seq_len, head_dim)
            assert cos_pos_embed.dim(1) == head_dim and sin_pos_embed.dim(1) == head_dim
            rotary_embed = 1
        qk_norm = 0
        if q_norm is not None or k_norm is not None:
            assert q_norm.num_dims == 1 and k_norm.num_dims == 1  # (head_dim)
            assert q_norm.dim(0) == head_dim and k_norm.dim(0) == head_dim
            qk_norm = 1
        return qk_norm, rotary_embed

    def paged_attention_layer(self, input: DTensor, k_cache: DTensor, v_cache: DTensor, q_norm: DTensor, k_norm: DTensor, cos_pos_embed: DTensor,
                              sin_pos_embed: DTensor, output: DTensor, grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:724: q/k-norm + RoPE + KV append + paged attention as one task."""
        assert input.num_dims == 2 and output.num_dims == 2
        assert k_cache.num_dims == 4 and v_cache.num_dims == 4  # (num_pages, page_size, kv_heads, head_dim)
        assert k_cache.dim(0) == self.max_num_pages and v_cache.dim(0) == self.max_num_pages
        assert k_cache.dim(1) == self.page_size and v_cache.dim(1) == self.page_size
        head_dim, num_kv_heads = k_cache.dim(3), k_cache.dim(2)
        num_q_heads = output.dim(1) // head_dim
        qk_norm, rotary_embed = self._attn_flags(q_norm, k_norm, cos_pos_embed, sin_pos_embed, head_dim)
        assert grid_dim[0] == self.max_num_batched_requests
        assert grid_dim[1] == num_kv_heads
        self._task("paged_attention", grid_dim, block_dim,
                   [(input, (-1, 1, -1), -1), (k_cache, (-1, 2, -1), 1), (v_cache, (-1, 2, -1), 1), (q_norm, _REPL, -1), (k_norm, _REPL, -1),
                    (cos_pos_embed, _REPL, -1), (sin_pos_embed, _REPL, -1), (output, (-1, 1, -1), -1)],
                   [num_q_heads, num_kv_heads, qk_norm, rotary_embed, self.max_seq_length, self.page_size])

    def paged_attention_split_kv_layer(self, input: DTensor, k_cache: DTensor, v_cache: DTensor, q_norm: DTensor, k_norm: DTensor,
                                       cos_pos_embed: DTensor, sin_pos_embed: DTensor, lse: DTensor, output: DTensor, attention_params: tuple,
                                       grid_dim: tuple, block_dim: tuple):
        """persistent_kernel.py:804.  Must be followed by paged_attention_split_kv_merge_layer over the same lse / output
        tensors: the pair becomes ONE attention stage, which chooses its own KV split (at least 64 positions per chunk, as
        many chunks as there are idle workgroups) and merges the chunks with the same rule (merge_splitkv.cuh:191-219).
        `lse` and the chunked `output` are never written."""
        assert input.num_dims == 2
        assert k_cache.num_dims == 4 and v_cache.num_dims == 4
        assert k_cache.dim(0) == self.max_num_pages and v_cache.dim(0) == self.max_num_pages
        assert k_cache.dim(1) == self.page_size and v_cache.dim(1) == self.page_size
        assert output.num_dims == 3 and lse.num_dims == 3
        head_dim, num_kv_heads = k_cache.dim(3), k_cache.dim(2)
        num_q_heads, num_kv_chunks = attention_params[0], attention_params[1]
        qk_norm, rotary_embed = self._attn_flags(q_norm, k_norm, cos_pos_embed, sin_pos_embed, head_dim)
        assert grid_dim[0] == self.max_num_batched_requests
        assert grid_dim[1] == num_kv_heads
        self._task("paged_attention_split_kv_mi300", grid_dim, block_dim,
                   [(input, (-1, 1, -1), -1), (k_cache, (-1, 2, -1), 1), (v_cache, (-1, 2, -1), 1), (q_norm, _REPL, -1), (k_norm, _REPL, -1),
                    (cos_pos_embed, _REPL, -1), (sin_pos_embed, _REPL, -1), (lse, (-1, 2, 1), -1), (output, (-1, 2, 1), -1)],
                   [num_q_heads, num_kv_heads, qk_norm, rotary_embed, self.max_seq_length, self.page_size, num_kv_chunks])

    def paged_attention_split_kv_merge_layer(self, lse: DTensor, output_tmp: DTensor, output: DTensor, attention_params: tuple, grid_dim: tuple,
                                             block_dim: tuple):
        """persistent_kernel.py:894 (see paged_attention_split_kv_layer)."""
        assert lse.num_dims == 3 and output_tmp.num_dims == 3 and output.num_dims == 2
        num_q_heads, head_dim = attention_params[0], attention_params[1]
        num_kv_heads = grid_dim[1]
        self._task("paged_attention_split_kv_merge_mi300", grid_dim, block_dim,
                   [(lse, (-1, 2, -1), -1), (output_tmp, (-1, 2, -1), -1), (output, (-1, 1, -1), -1)],
                   [num_q_heads // num_kv_heads, head_dim, self.max_seq_length, self.page_size, num_kv_heads])

    def paged_attention_ck_fmha_merge_layer(self, lse: DTensor, output_tmp: DTensor, output: DTensor, attention_params: tuple, grid_dim: tuple,
                                            block_dim: tuple):
        """persistent_kernel.py:1028: closes a paged_attention_ck_fmha_layer built with num_kv_chunks > 1 whose o_acc / lse_acc
        are `output_tmp` / `lse`; the pair (after kv_cache_update_layer) becomes one attention stage writing `output`."""
        assert lse.num_dims == 2 and output_tmp.num_dims == 2 and output.num_dims == 2
        num_q_heads, head_dim, num_kv_chunks, num_kv_heads = attention_params[0], attention_params[1], attention_params[2], attention_params[3]
        self._task("paged_attention_ck_fmha_merge_mi300", grid_dim, block_dim,
                   [(lse, _REPL, -1), (output_tmp, _REPL, -1), (output, _REPL, -1)],
                   [num_q_heads // num_kv_heads, head_dim, self.max_seq_length, self.page_size, num_kv_heads, num_kv_chunks])

    def gang_paged_attention_split_kv_merge_layer(self, lse: DTensor, output_tmp: DTensor, output: DTensor, attention_params: tuple,
                                                  block_dim: tuple = (256, 1, 1)):
        """persistent_kernel.py:1141: closes a gang_paged_attention_split_kv_layer built with num_kv_chunks > 1."""
        assert lse.num_dims == 2 and output_tmp.num_dims == 2 and output.num_dims == 2
        num_q_heads, head_dim, num_kv_heads, num_kv_chunks = attention_params[0], attention_params[1], attention_params[2], attention_params[3]
        total = self.max_num_batched_requests * num_kv_heads
        self._task("gang_attn_merge_mi300", (8, 1, 1), block_dim,
                   [(lse, _REPL, -1), (output_tmp, _REPL, -1), (output, _REPL, -1)],
                   [num_q_heads // num_kv_heads, head_dim, self.max_seq_length, self.page_size, num_kv_heads, math.ceil(total / 8), total, num_kv_chunks])

    # ------------------------------------------------------------------ compile / run
    def describe_program(self) -> str:
        return self._g.describe_program()

    def compile(self, **kwargs):
        """persistent_kernel.py:2404.  Lowers the recorded tasks and uploads descriptors; nothing is compiled at run time."""
        assert not self._is_compiled
        output_dir = kwargs.get("output_dir", None)
        # The library allocates its buffers (tile copies of the weights, intermediates, partial buffers) with hipMalloc,
        # next to torch's caching allocator: blocks torch only caches are handed back first, or a process that has
        # built and dropped large models before can run out of device memory with most of it unused.
        if torch.cuda.is_available():
            torch.cuda.empty_cache()
        self._g.compile()
        self._is_compiled = True
        if self._profiler_tensor is not None:
            self._attach_profiler()
        if output_dir is not None:
            import os
            os.makedirs(output_dir, exist_ok=True)
            res = self.kn_graph.generate_task_graph(1, 0)
            with open(os.path.join(output_dir, "task_graph.json"), "w") as f:
                f.write(res["json_file"])
            with open(os.path.join(output_dir, "stage_program.txt"), "w") as f:
                f.write(self.describe_program())

    @property
    def profiler_tensor(self):
        return self._profiler_tensor

    @profiler_tensor.setter
    def profiler_tensor(self, t):
        """A uint64 device tensor the kernel records begin/end of every stage of every iteration into (reference: the
        profiler_tensor constructor argument, persistent_kernel.py:2590-2600); None stops recording."""
        self._profiler_tensor = t
        if self._is_compiled:
            self._attach_profiler()

    def _attach_profiler(self):
        t = self._profiler_tensor
        if t is None:
            self._g.set_profiler(0, 0)
            self._profiler_attached = False
            return
        assert t.is_cuda and t.dtype in (torch.uint64, torch.int64) and t.dim() == 1 and t.is_contiguous(), "the profiler tensor is a flat uint64 device tensor"
        self._g.set_profiler(t.data_ptr(), t.numel())
        self._profiler_attached = True

    @staticmethod
    def _stream_ptr(stream):
        if stream is None:
            stream = torch.cuda.current_stream()
        if hasattr(stream, "cuda_stream"):
            return int(stream.cuda_stream)
        if isinstance(stream, int):
            return stream
        raise ValueError("Invalid stream object")

    def __call__(self, **kwargs):
        """persistent_kernel.py:2622: run every request to completion in one persistent launch (blocking)."""
        assert self._is_compiled, "call compile() first"
        sp = self._stream_ptr(kwargs.get("default_stream", None))
        self._g.launch(sp)
        if self.profiler_tensor is not None:
            self.export_profile()

    def export_profile(self, trace_name: str = None):
        """With a profiler tensor (reference: persistent_kernel.py:2644-2658): what the kernel recorded into it (every stage
        of every iteration since the tensor was attached or the requests were last initialised, as far as it had room) goes
        out as `<trace_name>.perfetto-trace` (default mirage_<rank>), the raw tensor beside it as `.pt`.  Returns the path."""
        from .profiler_persistent import export_to_perfetto_trace
        assert self.profiler_tensor is not None, "no profiler tensor was passed to the constructor"
        name = (trace_name or self.trace_name or f"mirage_{self.mpi_rank}") + ".perfetto-trace"
        export_to_perfetto_trace(self.profiler_tensor, name)
        torch.save(self.profiler_tensor.cpu(), name.replace(".perfetto-trace", ".pt"))
        return name

    def init_request_resources(self):
        """Reset step[], batch slots and the page ring (reference: init_request_func, persistent_kernel.py:63-68)."""
        self._g.init_requests()

    def run_steps(self, max_iterations: int, default_stream=None) -> bool:
        """Run at most `max_iterations` decode iterations; returns True when all requests have finished."""
        return self._g.launch_steps(self._stream_ptr(default_stream), int(max_iterations))

    def enqueue_steps(self, max_iterations: int, default_stream=None):
        self._g.enqueue_steps(self._stream_ptr(default_stream), int(max_iterations))

    def wait(self, default_stream=None) -> bool:
        return self._g.wait(self._stream_ptr(default_stream))

    def run_once(self, tok_slot, tok_pos, tok_first=None, default_stream=None):
        """Host-driven single pass over the stage program (onepass mode): row t belongs to batch slot tok_slot[t] at
        absolute position tok_pos[t]; paged_kv_indptr/indices must already describe each slot's pages."""
        n = len(tok_slot)
        if tok_first is None:
            tok_first, first = [], {}
            for t in range(n):
                if t > 0 and tok_slot[t] == tok_slot[t - 1]:
                    tok_first.append(tok_first[-1])
                else:
                    tok_first.append(t)
        self._g.run_once(self._stream_ptr(default_stream), [int(x) for x in tok_slot], [int(x) for x in tok_pos], [int(x) for x in tok_first])

    def repack_weights(self):
        """Refresh the library's matrix-core copies of the linear weights after attached weight tensors were overwritten
        (graphs with max_num_batched_tokens > 8 stream a tile-ordered copy made at compile time).  Not in the reference,
        whose kernels read the attached tensors in place."""
        self._g.repack_weights()

    def release_row_major_weights(self) -> list:
        """After compile() of a graph built with single_weight_copy: drop this object's references to the attached weight
        tensors the kernel will never read again (each now lives in its tile copy only) and return their names, so that a
        caller who drops its own references as well gets the memory back.  Without single_weight_copy nothing is released."""
        assert self._is_compiled, "compile() first"
        released = []
        for t in self._tensors:
            if t.torch_tensor is not None and self._g.tensor_releasable(t.id):
                released.append(t.name)
                t.torch_tensor = None
        return released

    def stats(self) -> dict:
        return self._g.stats()

    def stage_profile(self, workgroup: int = 0, raw: bool = False, marks: bool = False):
        """Per-stage timing of the last iteration on one virtual workgroup: list of (description, entered,
        barrier_satisfied, work_done, arrived) in microseconds relative to that workgroup's first stage (raw=True:
        100 MHz ticks, comparable across workgroups; 0 = stage skipped).  The last entry, "SCHEDULER", times the scheduler
        step that opened the iteration: (previous iteration complete, batch prepared [workgroup 0], batch published, 0).
        marks=True returns the four in-stage marks of a library built with -DMK_TRACE instead."""
        n = self.stats()["num_stages"] + 1
        rows = self._g.stage_ticks(int(workgroup), n, bool(marks))
        desc = self.describe_program().splitlines() + ["SCHEDULER"]
        if raw:
            return [(desc[i], *row) for i, row in enumerate(rows)]
        t0 = min(row[0] for row in rows[:-1] if row[0] > 0) if len(rows) > 1 else 0
        return [(desc[i], *[(x - t0) * 0.01 if x > 0 else -1.0 for x in row]) for i, row in enumerate(rows)]

    def finalize(self):
        assert not self.__finalized__
        if self._handle is not None:
            self._g.destroy()
            self._handle = None
        self.__finalized__ = True

    def __del__(self, _is_finalizing=sys.is_finalizing):
        if _is_finalizing():  # the HIP runtime may already be gone at interpreter shutdown: leave the memory to the OS
            return
        try:
            if not self.__finalized__:
                self.finalize()
        except Exception:
            pass


class _DevicePtr:
    """Minimal __cuda_array_interface__ holder so torch can view library-owned device memory without copying."""

    def __init__(self, ptr, nbytes, shape, dt, device, strides=None):
        typestr = {"bfloat16": "<u2", "float16": "<f2", "float32": "<f4", "int32": "<i4", "int64": "<i8", "uint64": "<u8"}[dt.name]
        self._dt = dt
        iface = {"shape": tuple(shape), "typestr": typestr, "data": (int(ptr), False), "version": 2}
        if strides is not None:
            iface["strides"] = tuple(int(s) * dt.size for s in strides)
        self.__cuda_array_interface__ = iface
