"""MPK: the serving-facing wrapper around PersistentKernel + a model graph builder.

Same role as the reference's wrapper (python/mirage/mpk/mpk.py:16-428): a caller (its vLLM integration, or a script)
fills an `MPKMetadata` with the mode, the batch limits, the ten meta tensors (or None to have them allocated) and either
a `MirageModelConfig` (weights, KV cache and rotary tables it owns) or a local checkpoint path; `build()` records the
model graph through the registered builder, `compile()` lowers and uploads it, `__call__()` launches: the whole offline
generation in "offline" mode, ONE pass over the batch the caller described in the meta tensors in "online_notoken" mode
(and returns the normalised final hidden state when the graph has no LM head, as the reference does, mpk.py:419-421).

What differs on the host: no MPI / multi-GPU set-up (one GPU), nothing is compiled at run time, checkpoints are local
directories (no hub access).
"""
import sys
from dataclasses import dataclass
from typing import Optional

import torch

from ..utils import get_configurations_from_gpu
from .model_registry import get_builder
from .models.graph_builder import MirageModelConfig
from .persistent_kernel import PersistentKernel
from .speculative import spec_decode_class


@dataclass
class MPKMetadata:
    # args
    mode: str = "offline"
    total_num_requests: int = 1
    num_remote_schedulers: int = 0
    max_seq_length: int = 0
    max_num_batched_requests: int = 0
    max_num_batched_tokens: int = 0
    max_num_pages: int = 0
    page_size: int = 0
    max_sm_num: int = 108
    device: str = "cuda"
    # model
    weight_from_model: bool = False
    model_name: Optional[str] = None
    model_path: Optional[str] = None
    # multi device support
    world_size: int = 1
    rank: int = 0
    num_workers: int = -1
    num_schedulers: int = -1
    # meta tensors
    step: Optional[torch.Tensor] = None
    tokens: Optional[torch.Tensor] = None
    input_tokens: Optional[torch.Tensor] = None
    output_tokens: Optional[torch.Tensor] = None
    num_new_tokens: Optional[torch.Tensor] = None
    prompt_lengths: Optional[torch.Tensor] = None
    qo_indptr_buffer: Optional[torch.Tensor] = None
    paged_kv_indptr_buffer: Optional[torch.Tensor] = None
    paged_kv_indices_buffer: Optional[torch.Tensor] = None
    paged_kv_last_page_len_buffer: Optional[torch.Tensor] = None
    # MirageModelConfig
    model_config: Optional[MirageModelConfig] = None
    # profiling
    profiling: bool = False
    profiler_tensor: Optional[torch.Tensor] = None
    trace_name: Optional[str] = None
    # spec decode config
    spec_decode: Optional[str] = None       # "promptlookup": builds `spec_decode_config` from the two numbers below (mpk.py:283-288)
    ngram_size: int = 3
    spec_length: int = 5
    spec_decode_config: Optional[object] = None
    use_cutlass_kernel: bool = False
    eos_token_id: Optional[int] = None
    max_tokens_per_request: Optional[int] = None
    single_weight_copy: Optional[bool] = None  # keep every linear weight once, in tile order (see PersistentKernel)

    def check_valid(self):
        if self.weight_from_model:
            assert (self.model_name is not None) or (self.model_path is not None), "model_name or model_path is required when weight_from_model is True"
        else:
            assert self.model_config is not None and self.model_config.state_dict is not None, "state_dict is required when weight_from_model is False"
            assert self.model_config.k_cache is not None, "k_cache is required when weight_from_model is False"
            assert self.model_config.v_cache is not None, "v_cache is required when weight_from_model is False"

    def info_as_string(self):
        shape = lambda t: None if t is None else tuple(t.shape)
        rows = [("Mode", self.mode), ("Total number of requests", self.total_num_requests), ("Max sequence length", self.max_seq_length),
                ("Max number of batched requests", self.max_num_batched_requests), ("Max number of batched tokens", self.max_num_batched_tokens),
                ("Max number of pages", self.max_num_pages), ("Page size", self.page_size), ("Device", self.device),
                ("Weight from model", self.weight_from_model), ("Model name", self.model_name), ("Model path", self.model_path),
                ("World size", self.world_size), ("Rank", self.rank), ("Step", shape(self.step)), ("Tokens", shape(self.tokens)),
                ("Input tokens", shape(self.input_tokens)), ("Output tokens", shape(self.output_tokens)),
                ("QO indptr buffer", shape(self.qo_indptr_buffer)), ("Paged KV indptr buffer", shape(self.paged_kv_indptr_buffer)),
                ("Paged KV indices buffer", shape(self.paged_kv_indices_buffer)),
                ("Paged KV last page len buffer", shape(self.paged_kv_last_page_len_buffer))]
        info = "MPKMetadata info:\n" + "".join(f"{k}: {v}\n" for k, v in rows)
        if self.model_config is not None:
            info += "Model config:\n" + self.model_config.info_as_string()
        return info

    def print_info(self):
        print(self.info_as_string())

    def write_to_file(self, file_path: str):
        """The same summary as print_info, into a text file (mpk.py:102-104)."""
        with open(file_path, "w") as f:
            f.write(self.info_as_string())


class MPK:
    def __init__(self, meta: MPKMetadata):
        if meta.world_size != 1 or meta.rank != 0:
            raise NotImplementedError("the MI355X megakernel runs on one GPU (world_size=1, rank=0)")
        meta.check_valid()
        self.metadata = meta
        self.world_size, self.rank = 1, 0
        self.model_name = meta.model_name or "Qwen3"
        self.device = meta.device
        self.weight_from_model = meta.weight_from_model
        self.max_seq_length = meta.max_seq_length
        self.max_num_batched_tokens = meta.max_num_batched_tokens
        self.max_num_batched_requests = meta.max_num_batched_requests
        self.max_num_pages = meta.max_num_pages
        # as the reference does (mpk.py:277): the request table has one row per batch slot
        self.total_num_requests = meta.max_num_batched_requests if meta.mode != "offline" else max(meta.total_num_requests, 1)
        self.tokenizer = None
        # the kernel reads int64 token ids; a caller that keeps int32 ids gets a staging tensor copied in at every call
        self.need_cpy_input, self.src_input_tokens = False, None
        self.step, self.tokens = meta.step, meta.tokens
        self.input_tokens = meta.input_tokens
        if meta.input_tokens is not None and meta.input_tokens.dtype != torch.int64:
            self.need_cpy_input, self.src_input_tokens = True, meta.input_tokens
            self.input_tokens = torch.empty_like(meta.input_tokens, dtype=torch.int64)
        self.output_tokens = meta.output_tokens
        self.num_new_tokens, self.prompt_lengths = meta.num_new_tokens, meta.prompt_lengths
        self.qo_indptr_buffer, self.paged_kv_indptr_buffer = meta.qo_indptr_buffer, meta.paged_kv_indptr_buffer
        self.paged_kv_indices_buffer, self.paged_kv_last_page_len_buffer = meta.paged_kv_indices_buffer, meta.paged_kv_last_page_len_buffer
        self.compensate_meta_tensors()
        self.model_config = meta.model_config
        self.with_lm_head = True if self.model_config is None else self.model_config.with_lm_head
        if meta.num_workers <= 0:
            dev = torch.device(self.device)
            self.num_workers, self.num_schedulers = get_configurations_from_gpu(dev.index if dev.index is not None else torch.cuda.current_device())
        else:
            self.num_workers, self.num_schedulers = meta.num_workers, max(meta.num_schedulers, 0)
        # `profiling` without a tensor of the caller's: one of the reference's size (mpk.py:276-279); the kernel fills it
        # from the first iteration on until it is full
        self.profiler_tensor = meta.profiler_tensor
        if meta.profiling and self.profiler_tensor is None:
            self.profiler_tensor = torch.zeros(3000 * 128, dtype=torch.uint64, device=self.device)
        if meta.spec_decode_config is None and meta.spec_decode:
            meta.spec_decode_config = spec_decode_class(meta.spec_decode, ngram_size=meta.ngram_size, spec_length=meta.spec_length)
        self.spec_decode_config = meta.spec_decode_config
        self.persistent_kernel = PersistentKernel(
            mode=meta.mode, world_size=1, mpi_rank=0, num_workers=self.num_workers, num_local_schedulers=self.num_schedulers,
            num_remote_schedulers=0, max_seq_length=self.max_seq_length, max_num_batched_requests=meta.max_num_batched_requests,
            max_num_batched_tokens=self.max_num_batched_tokens, max_num_pages=meta.max_num_pages, page_size=meta.page_size,
            meta_tensors={
                "step": self.step, "tokens": self.tokens, "input_tokens": self.input_tokens, "output_tokens": self.output_tokens,
                "num_new_tokens": self.num_new_tokens, "prompt_lengths": self.prompt_lengths, "qo_indptr_buffer": self.qo_indptr_buffer,
                "paged_kv_indptr_buffer": self.paged_kv_indptr_buffer, "paged_kv_indices_buffer": self.paged_kv_indices_buffer,
                "paged_kv_last_page_len_buffer": self.paged_kv_last_page_len_buffer},
            profiler_tensor=self.profiler_tensor, trace_name=meta.trace_name, spec_decode_config=meta.spec_decode_config,
            use_cutlass_kernel=False, eos_token_id=meta.eos_token_id if meta.eos_token_id is not None else 151645,
            max_tokens_per_request=meta.max_tokens_per_request, single_weight_copy=meta.single_weight_copy)
        self.is_built = self.task_graph_generated = self.is_compiled = False

    def compensate_meta_tensors(self):
        """Allocate the meta tensors the caller left out (mpk.py:229-267)."""
        R, B, T = self.max_num_batched_requests, self.max_num_batched_tokens, self.total_num_requests
        # name -> (shape, dtype, initial value); one new token per request per pass is the reference's default as well
        layout = {"step": ((T,), torch.int32, 0), "tokens": ((T, self.max_seq_length), torch.int64, 0),
                  "input_tokens": ((B, 1), torch.int64, 0), "output_tokens": ((B, 1), torch.int64, 0),
                  "num_new_tokens": ((T,), torch.int32, 1), "prompt_lengths": ((T,), torch.int32, 0),
                  "qo_indptr_buffer": ((R + 1,), torch.int32, 0), "paged_kv_indptr_buffer": ((R + 1,), torch.int32, 0),
                  "paged_kv_indices_buffer": ((self.max_num_pages,), torch.int32, 0), "paged_kv_last_page_len_buffer": ((R,), torch.int32, 0)}
        for name, (shape, dtype, fill) in layout.items():
            if getattr(self, name) is None:
                setattr(self, name, torch.full(shape, fill, dtype=dtype, device=self.device))
        self.total_num_requests = self.tokens.shape[0]

    # ------------------------------------------------------------------ requests
    def load_new_request(self, prompt, use_template: bool = True):
        """Every request slot gets `prompt` (mpk.py:281-307): a string (needs the checkpoint's tokenizer) or a 1-D sequence
        of token ids."""
        self._require_built()
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("no tokenizer was loaded with the model: pass token ids")
            if use_template:
                messages = [{"role": "system", "content": "You are Qwen, created by Alibaba Cloud. You are a helpful assistant."},
                            {"role": "user", "content": prompt}]
                prompt = self.tokenizer.apply_chat_template(messages, tokenize=False, add_generation_prompt=True)
            ids = self.tokenizer([prompt], return_tensors="pt").input_ids[0]
        else:
            ids = torch.as_tensor(prompt, dtype=torch.int64)
        L = ids.shape[-1]
        assert 0 < L < self.max_seq_length
        self.tokens.zero_()
        self.tokens[:, :L].copy_(ids.to(self.tokens.device).unsqueeze(0).expand(self.total_num_requests, -1))
        self.prompt_lengths.fill_(L)

    def clear_buffers(self):
        for t in (self.step, self.tokens, self.input_tokens, self.output_tokens, self.num_new_tokens, self.prompt_lengths, self.qo_indptr_buffer,
                  self.paged_kv_indptr_buffer, self.paged_kv_indices_buffer, self.paged_kv_last_page_len_buffer):
            t.fill_(0)

    def print_buffers(self, logger=None):
        """The ten meta tensors, to `logger.info` or to stdout (mpk.py:329-341)."""
        emit = logger.info if logger is not None else print
        for name in ("step", "tokens", "input_tokens", "output_tokens", "num_new_tokens", "prompt_lengths", "qo_indptr_buffer",
                     "paged_kv_indptr_buffer", "paged_kv_indices_buffer", "paged_kv_last_page_len_buffer"):
            emit(f"{name}: {getattr(self, name)}")

    def grid_dim_sanitizer(self, grid_dim):
        """Halve the last dimension that is still above one until the task grid fits `max_sm_num` workers
        (mpk.py:369-382).  The builders here size their grids from `num_workers` already; kept for callers that build
        layers by hand."""
        dims = list(grid_dim)
        limit = max(int(self.metadata.max_sm_num or 0), 1)
        while dims[0] * dims[1] * dims[2] > limit and any(d > 1 for d in dims):
            i = max(j for j in range(3) if dims[j] > 1)
            dims[i] //= 2
        return tuple(dims)

    def init_per_request(self):
        self.persistent_kernel.init_request_resources()

    init_request_func = init_per_request

    def run(self, prompt):
        """Offline generation of one prompt in every request slot; returns the decoded text (or the token ids when the
        model came without a tokenizer), mpk.py:336-349."""
        self._ensure_compiled()
        self.load_new_request(prompt)
        torch.cuda.synchronize()  # the prompt rows are in place before the request state is reset and the kernel starts
        self.init_per_request()
        self()
        torch.cuda.synchronize()
        rows = [self.tokens[r, : int(n) + 1] for r, n in enumerate(self.step.tolist())]
        if self.tokenizer is None:
            return [ids.cpu() for ids in rows]
        return [self.tokenizer.decode(ids, skip_special_tokens=True) for ids in rows]

    # ------------------------------------------------------------------ graph
    def _require_built(self):
        if not self.is_built:
            raise ValueError("the model graph is not built yet: call build() first")

    def _ensure_compiled(self):
        if not self.is_compiled:
            self.compile()

    def build(self):
        """Record the model graph through the builder registered for the model name (mpk.py:351-367)."""
        self.model_builder = get_builder(self.model_name or "Qwen3")(self.persistent_kernel)
        if not self.weight_from_model:
            self.model_builder.build_from_config(self.model_config)
        else:
            self.model_builder.build_from_model(model_name=self.metadata.model_name, model_path=self.metadata.model_path)
            self.tokenizer = self.model_builder.tokenizer
        self.with_lm_head = self.model_builder.with_lm_head
        self.is_built = True

    def generate_task_graph(self):
        self._require_built()
        self.task_graph_generated = True
        return self.persistent_kernel.kn_graph.generate_task_graph(num_gpus=1, my_gpu_id=0)

    def compile(self, output_dir: str = None):
        self._require_built()
        self.persistent_kernel.compile(output_dir=output_dir)
        self.is_compiled = True
        if self.persistent_kernel.single_weight_copy:
            # the row-major tensors of the linears now exist in tile order inside the library: drop them here and in the
            # builder (a state dict the caller still holds keeps its tensors alive until the caller lets go)
            self.model_builder.release_weights(self.persistent_kernel.release_row_major_weights())

    def __call__(self, **kwargs):
        """One launch (mpk.py:405-421).  Returns the normalised last hidden state when the graph was built without an LM
        head and the caller drives single passes, None otherwise."""
        self._ensure_compiled()
        if self.src_input_tokens is not None:  # the caller's ids are not int64: refresh the staging copy the kernel reads
            self.input_tokens.copy_(self.src_input_tokens)
        self.persistent_kernel(**kwargs)
        headless_pass = self.persistent_kernel.mode == "online_notoken" and not self.with_lm_head
        return self.model_builder.returned_hidden_state if headless_pass else None

    def decode(self, ids: torch.Tensor):
        return self.model_builder.decode(ids)

    def finalize(self):
        self.persistent_kernel.finalize()

    def __del__(self, _is_finalizing=sys.is_finalizing):
        # the reference finalizes in its destructor (mpk.py:426-429); a kernel the caller finalized already is left alone
        pk = getattr(self, "persistent_kernel", None)
        if pk is not None and not _is_finalizing() and not getattr(pk, "__finalized__", True):
            try:
                pk.finalize()
            except Exception:
                pass
