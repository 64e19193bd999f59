"""Qwen3 graph builder: replays a Qwen3 decoder onto a PersistentKernel from a state dict.

Same role and entry points as the reference's builder (python/mirage/mpk/models/qwen3/builder.py:13-824):
`build_from_config(MirageModelConfig)` for a caller that owns the weights, KV cache and rotary tables (the serving
integration), `build_from_model(model_name, model_path)` for a local checkpoint directory, `build_from_dict` underneath.
The layer sequence is the one that builder emits for this GPU family (its `target_cc == 94` branches, :395-420,
:560-585, :700-712): rmsnorm -> split-K linear into an fp32 workspace + split-K reduce (QKV, with a zero residual) ->
kv_cache_update + attention (or the fused paged attention task) -> split-K linear + reduce with the residual (o_proj) ->
rmsnorm -> linear (gate/up, interleaved in groups) -> silu_mul_linear_with_residual (down_proj) -> final rmsnorm ->
LM head -> argmax partial / reduce.  Every one of those tasks lowers to the megakernel's stage program.

Differences from the reference builder, all on the host side: interleaved QKV and gate/up weights are views
(`shuffle_tensors`), never copies -- also in online_notoken mode, where the reference materialises them (:337-351);
the LM head is not padded to 153,600 rows (:744-756: any row count works); checkpoints are read from local safetensors
files only (there is no hub access here), through `checkpoint.load_checkpoint`.
"""
import os
from typing import Optional

import torch

from ...model_registry import register_model_builder
from ...persistent_kernel import PersistentKernel
from ....kernel import bfloat16, int64
from ..graph_builder import GraphBuilder, MirageModelConfig
from ..utils import grid_for_rmsnorm_linear_layer


@register_model_builder("Qwen3", "Qwen/Qwen3-8B", "Qwen/Qwen3-1.7B", "Qwen/Qwen3-14B", "Qwen/Qwen3-0.6B")
class Qwen3Builder(GraphBuilder):
    def __init__(self, mpk: PersistentKernel, weights: Optional[dict] = None):
        super().__init__(mpk, weights)
        self.max_num_pages = mpk.max_num_pages
        self.page_size = mpk.page_size
        self.world_size = mpk.world_size
        self.input_tokens = mpk.meta_tensors["input_tokens"]
        self.output_tokens = mpk.meta_tensors["output_tokens"]
        self.tokenizer = None
        self.model_name = None
        self.model_path = None
        self.rank = mpk.mpi_rank
        self.eos_token_id = 151645  # default eos token id for Qwen3 (builder.py:27)
        self.returned_hidden_state = None
        self._keep = []
        self._kept_as = {}  # torch tensors the graph points at

    # ------------------------------------------------------------------ entry points
    def build_from_config(self, model_config: MirageModelConfig):
        self.position_embeddings = model_config.position_embeddings
        self.k_cache = model_config.k_cache
        self.v_cache = model_config.v_cache
        self.hidden_size = model_config.hidden_size
        self.intermediate_size = model_config.intermediate_size
        self.vocab_size = model_config.vocab_size
        self.num_local_q_heads = model_config.local_num_q_heads
        self.num_local_kv_heads = model_config.local_num_kv_heads
        self.head_dim = model_config.head_dim
        self.num_layers = model_config.num_layers
        self._derived()
        self.build_from_dict(model_config.state_dict, model_config.with_lm_head)

    def build_from_model(self, model_name: str = None, model_path: str = None):
        """Build from a LOCAL checkpoint directory (config.json + *.safetensors [+ tokenizer files]).  `model_name` alone
        would mean a hub download, which this environment cannot do: it raises."""
        from .. import checkpoint
        if model_path is None:
            raise ValueError(f"model '{model_name}': a local model_path is required (no hub access); it must hold config.json and *.safetensors")
        self.model_name, self.model_path = model_name, model_path
        cfg, state_dict = checkpoint.load_checkpoint(model_path, device=self.mpk.device, rank=self.rank, world_size=self.world_size)
        self.config = cfg
        self.hidden_size = cfg["hidden_size"]
        self.intermediate_size = cfg["intermediate_size"]
        self.vocab_size = cfg["vocab_size"]
        self.num_local_q_heads = cfg["num_attention_heads"] // self.world_size
        self.num_local_kv_heads = cfg["num_key_value_heads"] // self.world_size
        self.head_dim = cfg.get("head_dim") or self.hidden_size // cfg["num_attention_heads"]
        self.num_layers = cfg["num_hidden_layers"]
        if cfg.get("eos_token_id") is not None:
            eos = cfg["eos_token_id"]
            self.eos_token_id = eos[0] if isinstance(eos, (list, tuple)) else eos
        self.tokenizer = checkpoint.load_tokenizer(model_path)
        theta = cfg.get("rope_theta") or (cfg.get("rope_parameters") or {}).get("rope_theta", 1e6)
        n_pos = max(self.mpk.max_seq_length, 16)
        self.position_embeddings = checkpoint.rotary_tables(self.head_dim, theta, n_pos, self.mpk.device)
        dev = self.mpk.device
        shape = (self.num_layers, self.max_num_pages, self.page_size, self.num_local_kv_heads, self.head_dim)
        self.k_cache = torch.zeros(shape, dtype=torch.bfloat16, device=dev)
        self.v_cache = torch.zeros(shape, dtype=torch.bfloat16, device=dev)
        self._derived()
        if "lm_head.weight" not in state_dict and cfg.get("tie_word_embeddings"):
            state_dict["lm_head.weight"] = state_dict["model.embed_tokens.weight"]
        self.build_from_dict(state_dict, True)

    def _derived(self):
        self.fused_outdim_1 = (self.num_local_q_heads + 2 * self.num_local_kv_heads) * self.head_dim
        self.fused_outdim_2 = 2 * self.intermediate_size

    # ------------------------------------------------------------------ tensors
    def _attach(self, t: torch.Tensor, name: str):
        self._keep.append(t)
        self._kept_as[name] = t
        return self.mpk.attach_input(torch_tensor=t, name=name)

    def release_weights(self, names):
        """Drop this builder's references to the attached tensors `names` (those the compiled kernel no longer reads: a
        graph built with single_weight_copy keeps its linear weights in tile order only)."""
        gone = [self._kept_as.pop(n) for n in names if n in self._kept_as]
        self._keep = [t for t in self._keep if not any(t is g for g in gone)]
        return len(gone)

    def new_intermediate_tensors(self):
        """Activations of one iteration.  In online_notoken mode they are torch tensors the caller can read back (the
        normalised final hidden state is `returned_hidden_state`, as in the reference builder :120-126); otherwise they
        are owned by the library."""
        mpk, B = self.mpk, self.mpk.max_num_batched_tokens
        self.max_num_batched_tokens = B
        dev = mpk.device
        fixed = mpk.mode == "online_notoken"

        def act(name, cols, dt=bfloat16):
            if fixed:
                return self._attach(torch.zeros(B, cols, dtype=dt.torch_dtype, device=dev), name)
            return mpk.new_tensor(dims=(B, cols), dtype=dt, name=name, io_category="cuda_tensor")

        self.y = act("embed_out", self.hidden_size)
        if fixed:
            self.returned_hidden_state = torch.zeros(B, self.hidden_size, dtype=torch.bfloat16, device=dev)
            self.rmsnorm_out = self._attach(self.returned_hidden_state, "rmsnorm_out")
        else:
            self.rmsnorm_out = act("rmsnorm_out", self.hidden_size)
        self.attn_in = act("attn_in", self.fused_outdim_1)
        self.attn_out = act("attn_out", self.num_local_q_heads * self.head_dim)
        self.attn_proj_out = act("attn_proj_out", self.hidden_size)
        self.mlp_mid = act("mlp_mid", self.fused_outdim_2)
        self.silu_mul_out = act("silu_mul_out", self.intermediate_size)
        self.mlp_out = act("mlp_out", self.hidden_size)
        if self.with_lm_head:
            self.argmax_in = act("argmax_in", self.vocab_size)
            self.argmax_part_value = act("argmax_part_value", mpk.num_workers)
            self.argmax_part_index = act("argmax_part_index", mpk.num_workers, int64)

    # ------------------------------------------------------------------ layers
    def build_layers(self, state_dict: dict):
        mpk, B = self.mpk, self.mpk.max_num_batched_tokens
        dev = mpk.device
        H, D = self.hidden_size, self.head_dim
        nq, nkv = self.num_local_q_heads, self.num_local_kv_heads
        # split-K bookkeeping as the reference builder does it (:263-286): k_sp slices of 128-wide K tiles
        k_tiles_o = (nq * D) // 128
        self.splitk_k_sp = min(4, k_tiles_o)
        while k_tiles_o % self.splitk_k_sp != 0 and self.splitk_k_sp > 1:
            self.splitk_k_sp -= 1
        k_sp = self.splitk_k_sp
        self.splitk_ws = self._attach(torch.zeros(k_sp * B, H, dtype=torch.float32, device=dev), "splitk_workspace")
        self.splitk_ws_qkv = self._attach(torch.zeros(k_sp * B, self.fused_outdim_1, dtype=torch.float32, device=dev), "splitk_workspace_qkv")
        self.qkv_zero_res = self._attach(torch.zeros(B, self.fused_outdim_1, dtype=torch.bfloat16, device=dev), "qkv_zero_residual")
        self.use_ck_fmha = int(os.environ.get("USE_CK_FMHA", "0")) == 1
        if self.use_ck_fmha:
            self.ck_fmha_num_kv_chunks = int(os.environ.get("CK_FMHA_KV_CHUNKS", "1"))
            qpk, ch = nq // nkv, self.ck_fmha_num_kv_chunks
            self.ck_fmha_q_ws = self._attach(torch.zeros(B, nq * D, dtype=torch.bfloat16, device=dev), "ck_fmha_q_workspace")
            self.ck_fmha_o_acc = self._attach(torch.zeros(B, nkv * ch * qpk * D, dtype=torch.float32, device=dev), "ck_fmha_o_acc")
            self.ck_fmha_lse_acc = self._attach(torch.zeros(B, nkv * ch * qpk, dtype=torch.float32, device=dev), "ck_fmha_lse_acc")
        for i in range(self.num_layers):
            prefix = f"model.layers.{i}."
            w_norm = self._attach(state_dict[f"{prefix}input_layernorm.weight"], f"layer_{i}_input_layernorm")
            if f"{prefix}self_attn.q_proj.weight" in state_dict:
                w_q = self._attach(state_dict[f"{prefix}self_attn.q_proj.weight"], f"layer_{i}_q_proj")
                w_k = self._attach(state_dict[f"{prefix}self_attn.k_proj.weight"], f"layer_{i}_k_proj")
                w_v = self._attach(state_dict[f"{prefix}self_attn.v_proj.weight"], f"layer_{i}_v_proj")
                w_qkv = mpk.shuffle_tensors(inputs=[w_q, w_k, w_v], shuffled_dim=0, num_groups=nkv, name=f"layer_{i}_qkv_proj")
            elif f"{prefix}self_attn.qkv_proj.weight" in state_dict:  # already interleaved per kv head by the caller
                w_qkv = self._attach(state_dict[f"{prefix}self_attn.qkv_proj.weight"], f"layer_{i}_qkv_proj")
            else:
                raise ValueError(f"No qkv projection weight found for layer {i}")
            mpk.rmsnorm_layer(input=self.x, weight=w_norm, output=self.rmsnorm_out, grid_dim=(B, 1, 1), block_dim=(128, 1, 1))
            output_size = w_qkv.dim(0)
            assert output_size % 128 == 0, f"QKV output_size={output_size} not divisible by 128"
            mpk.splitk_linear_layer(input=self.rmsnorm_out, weight=w_qkv, output=self.splitk_ws_qkv, grid_dim=(output_size // 128, k_sp, 1),
                                    block_dim=(256, 1, 1))
            mpk.splitk_reduce_layer(workspace=self.splitk_ws_qkv, residual=self.qkv_zero_res, output=self.attn_in, k_splits=k_sp,
                                    grid_dim=(output_size // 128, 1, 1), block_dim=(256, 1, 1))
            w_q_norm = self._attach(state_dict[f"{prefix}self_attn.q_norm.weight"], f"layer_{i}_q_norm")
            w_k_norm = self._attach(state_dict[f"{prefix}self_attn.k_norm.weight"], f"layer_{i}_k_norm")
            k_cache = self._attach(self.k_cache[i], f"layer_{i}_k_cache")
            v_cache = self._attach(self.v_cache[i], f"layer_{i}_v_cache")
            R = mpk.max_num_batched_requests
            if self.use_ck_fmha:
                mpk.kv_cache_update_layer(input=self.attn_in, k_cache=k_cache, v_cache=v_cache, q_norm=w_q_norm, k_norm=w_k_norm,
                                          cos_pos_embed=self.cos_pos_embed, sin_pos_embed=self.sin_pos_embed, q_workspace=self.ck_fmha_q_ws,
                                          grid_dim=(R, nkv, 1), block_dim=(256, 1, 1))
                ch = self.ck_fmha_num_kv_chunks
                mpk.paged_attention_ck_fmha_layer(q_workspace=self.ck_fmha_q_ws, k_cache=k_cache, v_cache=v_cache,
                                                  o_acc=self.attn_out if ch == 1 else self.ck_fmha_o_acc, lse_acc=self.ck_fmha_lse_acc,
                                                  attention_params=(nq, ch, R), grid_dim=(R, nkv, ch), block_dim=(256, 1, 1))
                if ch > 1:
                    mpk.paged_attention_ck_fmha_merge_layer(lse=self.ck_fmha_lse_acc, output_tmp=self.ck_fmha_o_acc, output=self.attn_out,
                                                            attention_params=(nq, D, ch, nkv), grid_dim=(R, nkv, 1), block_dim=(256, 1, 1))
            else:
                mpk.paged_attention_layer(input=self.attn_in, k_cache=k_cache, v_cache=v_cache, q_norm=w_q_norm, k_norm=w_k_norm,
                                          cos_pos_embed=self.cos_pos_embed, sin_pos_embed=self.sin_pos_embed, output=self.attn_out,
                                          grid_dim=(R, nkv, 1), block_dim=(128, 1, 1))
            w_o = self._attach(state_dict[f"{prefix}self_attn.o_proj.weight"], f"layer_{i}_o_proj")
            mpk.splitk_linear_layer(input=self.attn_out, weight=w_o, output=self.splitk_ws, grid_dim=(H // 128, k_sp, 1), block_dim=(256, 1, 1))
            mpk.splitk_reduce_layer(workspace=self.splitk_ws, residual=self.x, output=self.attn_proj_out, k_splits=k_sp,
                                    grid_dim=(H // 128, 1, 1), block_dim=(256, 1, 1))
            self.x = self.attn_proj_out
            w_norm2 = self._attach(state_dict[f"{prefix}post_attention_layernorm.weight"], f"layer_{i}_post_attn_layernorm")
            gate_rows = None  # a shuffled view knows its own groups; a weight the caller interleaved needs them spelt out
            if f"{prefix}mlp.gate_proj.weight" in state_dict:
                rmsnorm_num_tasks = grid_for_rmsnorm_linear_layer(2 * state_dict[f"{prefix}mlp.gate_proj.weight"].shape[0])
                w_gate = self._attach(state_dict[f"{prefix}mlp.gate_proj.weight"], f"layer_{i}_gate_proj")
                w_up = self._attach(state_dict[f"{prefix}mlp.up_proj.weight"], f"layer_{i}_up_proj")
                w_gatedup = mpk.shuffle_tensors(inputs=[w_gate, w_up], shuffled_dim=0, num_groups=rmsnorm_num_tasks // 2, name=f"layer_{i}_gatedup_proj")
            elif f"{prefix}mlp.gate_up_proj.weight" in state_dict:  # already interleaved in rmsnorm_num_tasks / 2 groups by the caller
                rmsnorm_num_tasks = grid_for_rmsnorm_linear_layer(state_dict[f"{prefix}mlp.gate_up_proj.weight"].shape[0])
                w_gatedup = self._attach(state_dict[f"{prefix}mlp.gate_up_proj.weight"], f"layer_{i}_gatedup_proj")
                gate_rows = state_dict[f"{prefix}mlp.gate_up_proj.weight"].shape[0] // rmsnorm_num_tasks
            else:
                raise ValueError(f"No gate or up projection weight found for layer {i}")
            mpk.rmsnorm_layer(input=self.x, weight=w_norm2, output=self.rmsnorm_out, grid_dim=(B, 1, 1), block_dim=(128, 1, 1))
            mpk.linear_layer(input=self.rmsnorm_out, weight=w_gatedup, output=self.mlp_mid, grid_dim=(rmsnorm_num_tasks, 1, 1), block_dim=(128, 1, 1))
            w_down = self._attach(state_dict[f"{prefix}mlp.down_proj.weight"], f"layer_{i}_down_proj")
            mpk.silu_mul_linear_with_residual_layer(input=self.mlp_mid, weight=w_down, residual=self.x, output=self.mlp_out,
                                                    grid_dim=(H // 64, 1, 1), block_dim=(256, 1, 1), gate_rows_per_group=gate_rows)
            self.x = self.mlp_out

    def build_from_dict(self, state_dict: dict, with_lm_head: bool):
        mpk, B = self.mpk, self.mpk.max_num_batched_tokens
        self.with_lm_head = with_lm_head
        self.x = self._attach(self.input_tokens, "input_token")
        # prompt lookup (what the reference's builder leaves as a TODO at builder.py:719-745,811-816 and its llama demo
        # does, demo/llama3/demo.py:760-821): the n-gram tasks write the ids the embedding reads, a verify task follows
        # the sampling
        spec, spec_tokens = mpk.spec_decode_config, None
        if spec is not None:
            all_tokens = self._attach(mpk.meta_tensors["tokens"], "all_tokens")
            spec_tokens = mpk.draft_forward_layer_dispatcher(spec_decode_config=spec, tokens=all_tokens, grid_dim=(96, 1, 1), block_dim=(128, 1, 1))
            self.x = spec_tokens
        cos, sin = self.position_embeddings
        n_pos = min(cos.shape[-2], 4096) if cos.dim() == 3 else cos.shape[0]
        cos2 = (cos[0, :n_pos, :] if cos.dim() == 3 else cos).contiguous()
        sin2 = (sin[0, :n_pos, :] if sin.dim() == 3 else sin).contiguous()
        self.cos_pos_embed = self._attach(cos2, "cos_position_embedding")
        self.sin_pos_embed = self._attach(sin2, "sin_position_embedding")
        self.new_intermediate_tensors()
        argmax_out = self._attach(self.output_tokens, "output_token")
        w_embed = self._attach(state_dict["model.embed_tokens.weight"], "embed_tokens")
        mpk.embed_layer(input=self.x, weight=w_embed, output=self.y, grid_dim=(1, 1, 1), block_dim=(128, 1, 1), input_source=1)
        self.x = self.y
        self.build_layers(state_dict)
        w_norm = self._attach(state_dict["model.norm.weight"], "model_norm_weight")
        mpk.rmsnorm_layer(input=self.x, weight=w_norm, output=self.rmsnorm_out, grid_dim=(B, 1, 1), block_dim=(128, 1, 1))
        if self.with_lm_head:
            w_proj = self._attach(state_dict["lm_head.weight"], "lm_head")
            mpk.linear_layer(input=self.rmsnorm_out, weight=w_proj, output=self.argmax_in,
                             grid_dim=(grid_for_rmsnorm_linear_layer(w_proj.dim(0)), 1, 1), block_dim=(128, 1, 1))
            mpk.argmax_partial_layer(input=self.argmax_in, output=(self.argmax_part_value, self.argmax_part_index),
                                     grid_dim=(mpk.num_workers, 1, 1), block_dim=(128, 1, 1))
            mpk.argmax_reduce_layer(input=(self.argmax_part_value, self.argmax_part_index), output=argmax_out, grid_dim=(1, 1, 1),
                                    block_dim=(128, 1, 1))
            if spec_tokens is not None:
                self.verify_out = mpk.verify_layer_dispatcher(spec_decode_config=spec, spec_tokens=spec_tokens, target_output=argmax_out)
        elif spec_tokens is not None:
            raise ValueError("speculative decoding needs the LM head and the sampling stages in the graph (with_lm_head)")

    # ------------------------------------------------------------------ tokenizer pass-through
    def encode(self, text: str):
        return self.tokenizer.encode(text, add_special_tokens=True)

    def decode(self, ids: torch.Tensor):
        return self.tokenizer.decode(ids, skip_special_tokens=True)
