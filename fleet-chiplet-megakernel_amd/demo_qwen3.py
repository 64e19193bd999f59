"""Qwen3 decode driver (dense Qwen3-8B shape and mixture-of-experts Qwen3-30B-A3B shape) on the MI355X megakernel.

Builds the per-layer task graph through the PersistentKernel API the same way the reference driver
does (demo/qwen3/demo.py:314-1169), in either of its two README configurations:

* mode="fleet": gang tasks -- gang_rmsnorm -> gang_linear(QKV) -> gang attention (KV append + q/k norm +
  RoPE + attention) -> gang_linear_res(o) -> gang_rmsnorm -> gang_linear_silu(gate/up) -> gang_linear_res(down)
  (USE_GANG=1 USE_CK_FMHA=1 USE_FUSED_SILU=1, demo.py:556-1113);
* mode="mpk": rmsnorm -> linear -> kv_cache_update -> paged_attention_ck_fmha -> linear_with_residual ->
  rmsnorm -> linear -> silu_mul -> linear_with_residual (the non-gang path with separate activation).

With Qwen3Shape.num_experts > 0 the MLP is the reference's mixture-of-experts sequence (demo/qwen3/demo_30B_A3B.py:
675-754): router linear -> top-k softmax routing -> W13 per-expert linear -> SwiGLU -> W2 per-expert linear -> weighted
sum + residual ("fleet": the gang_moe_* layers, "mpk": the moe_* layers with explicit grids).

Both lower to the same stage program.  Weights are random-init (there is no checkpoint loader here);
the CLI prints decode ms/token measured over decode iterations only.
"""
import argparse
import math
import time
from dataclasses import dataclass

import torch

import mirage as mi


@dataclass
class Qwen3Shape:
    hidden_size: int = 4096
    num_q_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 12288
    num_layers: int = 36
    vocab_size: int = 151936
    rope_theta: float = 1e6
    num_experts: int = 0           # > 0: mixture-of-experts MLP
    num_experts_per_tok: int = 0
    moe_intermediate_size: int = 0

    @staticmethod
    def qwen3_30b_a3b(num_layers: int = 48):
        """Qwen3-30B-A3B: 48 layers, hidden 2048, 32 q / 4 kv heads, 128 experts, top-8, expert width 768."""
        return Qwen3Shape(hidden_size=2048, num_q_heads=32, num_kv_heads=4, head_dim=128, intermediate_size=0, num_layers=num_layers,
                          num_experts=128, num_experts_per_tok=8, moe_intermediate_size=768)

    def weight_bytes_per_token(self, distinct_experts: int = None):
        """bf16 weight bytes one decode step streams (all linears + LM head).  For the mixture-of-experts shape the
        expert term counts `distinct_experts` experts per layer (default: top-k, i.e. one token)."""
        H, I = self.hidden_size, self.intermediate_size
        qkv = (self.num_q_heads + 2 * self.num_kv_heads) * self.head_dim * H
        if self.num_experts > 0:
            ne = self.num_experts_per_tok if distinct_experts is None else distinct_experts
            mlp = self.num_experts * H + ne * 3 * self.moe_intermediate_size * H
        else:
            mlp = 2 * I * H + H * I
        per_layer = qkv + self.num_q_heads * self.head_dim * H + mlp
        return 2 * (self.num_layers * per_layer + self.vocab_size * H)

    def kv_bytes_per_position(self):
        """bf16 K+V bytes read per cached position per request per decode step (all layers)."""
        return self.num_layers * 2 * self.num_kv_heads * self.head_dim * 2


def random_weights(shape: Qwen3Shape, seed: int = 0, device="cuda"):
    """Random-init weights generated directly on the device: linears and embedding ~ N(0, 0.02), norm weights 1
    (what the reference's `_init_weights` gives, demo/qwen3/models/modeling_qwen3.py:404-413)."""
    g = torch.Generator(device=device).manual_seed(seed)
    H, I, D = shape.hidden_size, shape.intermediate_size, shape.head_dim

    def lin(n, k):
        w = torch.empty(n, k, dtype=torch.bfloat16, device=device)
        w.normal_(0.0, 0.02, generator=g)
        return w

    ones = lambda n: torch.ones(n, dtype=torch.bfloat16, device=device)
    w = {"embed": lin(shape.vocab_size, H), "layers": []}
    for _ in range(shape.num_layers):
        lw = {"input_norm": ones(H), "q_proj": lin(shape.num_q_heads * D, H), "k_proj": lin(shape.num_kv_heads * D, H),
              "v_proj": lin(shape.num_kv_heads * D, H), "q_norm": ones(D), "k_norm": ones(D), "o_proj": lin(H, shape.num_q_heads * D),
              "post_norm": ones(H)}
        if shape.num_experts > 0:
            E, MI = shape.num_experts, shape.moe_intermediate_size
            # packed per expert as the reference driver does (demo/qwen3/demo_30B_A3B.py:376-420): [gate ; up] rows
            lw.update({"router": lin(E, H), "gate_up_proj": lin(E * 2 * MI, H).view(E, 2 * MI, H), "down_proj": lin(E * H, MI).view(E, H, MI)})
        else:
            lw.update({"gate_proj": lin(I, H), "up_proj": lin(I, H), "down_proj": lin(H, I)})
        w["layers"].append(lw)
    w["final_norm"] = ones(H)
    w["lm_head"] = lin(shape.vocab_size, H)
    return w


def rope_tables(shape: Qwen3Shape, n_pos: int, device="cuda"):
    """bf16 cos/sin [n_pos, head_dim], both halves equal; fp32 math then cast
    (demo/qwen3/models/modeling_qwen3.py:100-117)."""
    D = shape.head_dim
    inv_freq = 1.0 / (shape.rope_theta ** (torch.arange(0, D, 2, dtype=torch.float32, device=device) / D))
    freqs = torch.arange(n_pos, dtype=torch.float32, device=device)[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(torch.bfloat16).contiguous(), emb.sin().to(torch.bfloat16).contiguous()


class Qwen3Decoder:
    """Owns the meta tensors, KV cache and PersistentKernel for one model; `generate` runs the persistent kernel."""

    def __init__(self, shape: Qwen3Shape, weights: dict, max_num_batched_tokens: int = 1, max_num_batched_requests: int = None,
                 max_seq_length: int = 1200, page_size: int = 4096, max_num_pages: int = None, total_requests: int = None,
                 mode: str = "fleet", eos_token_id: int = 0x7FFFFFFF, cos_sin=None, device="cuda", num_workers=None, with_head: bool = True,
                 kernel_mode: str = "offline", max_tokens_per_request: int = None, tap_last_layer_input: bool = False,
                 single_weight_copy: bool = None, spec_decode_config=None):
        assert mode in ("fleet", "mpk")
        self.shape, self.w, self.mode = shape, weights, mode
        self.with_head = with_head
        # (diagnostics) keep a copy of the hidden state entering the last layer in t["layer_in_tap"]: every layer writes the
        # same activation buffers, so the last layer otherwise overwrites its own input
        self.tap_last_layer_input = tap_last_layer_input
        B = max_num_batched_tokens
        R = max_num_batched_requests or B
        self.B, self.R = B, R
        self.max_seq = max_seq_length
        self.page_size = page_size
        pages_per_req = (max_seq_length + page_size - 1) // page_size
        self.max_pages = max_num_pages or R * pages_per_req
        self.total_requests = total_requests or R
        dev = device
        T = self.total_requests
        self.meta = {
            "step": torch.zeros(T, dtype=torch.int32, device=dev),
            "tokens": torch.zeros(T, max_seq_length, dtype=torch.int64, device=dev),
            "input_tokens": torch.zeros(B, 1, dtype=torch.int64, device=dev),
            "output_tokens": torch.zeros(B, 1, dtype=torch.int64, device=dev),
            "num_new_tokens": torch.ones(T, dtype=torch.int32, device=dev),
            "prompt_lengths": torch.zeros(T, dtype=torch.int32, device=dev),
            "qo_indptr_buffer": torch.zeros(R + 1, dtype=torch.int32, device=dev),
            "paged_kv_indptr_buffer": torch.zeros(R + 1, dtype=torch.int32, device=dev),
            "paged_kv_indices_buffer": torch.zeros(self.max_pages, dtype=torch.int32, device=dev),
            "paged_kv_last_page_len_buffer": torch.zeros(R, dtype=torch.int32, device=dev),
        }
        if num_workers is None:
            num_workers, _ = mi.get_configurations_from_gpu(torch.cuda.current_device())
        self.mpk = mi.PersistentKernel(
            mode=kernel_mode, world_size=1, mpi_rank=0, num_workers=num_workers, num_local_schedulers=0, num_remote_schedulers=0,
            max_seq_length=max_seq_length, max_num_batched_requests=R, max_num_batched_tokens=B, max_num_pages=self.max_pages,
            page_size=page_size, eos_token_id=eos_token_id, meta_tensors=self.meta, profiler_tensor=None, trace_name=None,
            spec_decode_config=spec_decode_config, use_cutlass_kernel=False, max_tokens_per_request=max_tokens_per_request,
            single_weight_copy=single_weight_copy)
        n_pos = max(max_seq_length, 16)
        self.cos, self.sin = cos_sin if cos_sin is not None else rope_tables(shape, n_pos, dev)
        L = shape.num_layers
        self.k_cache = torch.zeros(L, self.max_pages, page_size, shape.num_kv_heads, shape.head_dim, dtype=torch.bfloat16, device=dev)
        self.v_cache = torch.zeros_like(self.k_cache)
        self.t = {}
        self._build()
        self.mpk.compile()

    # graph construction, following demo/qwen3/demo.py:345-1169
    def _build(self):
        s, w, mpk, B = self.shape, self.w, self.mpk, self.B
        H, I, D = s.hidden_size, s.intermediate_size, s.head_dim
        nq, nkv = s.num_q_heads, s.num_kv_heads
        fused1 = (nq + 2 * nkv) * D
        gang = self.mode == "fleet"
        t = self.t
        x = mpk.attach_input(self.meta["input_tokens"], "input_token")
        spec, spec_tokens = mpk.spec_decode_config, None
        if spec is not None:
            # prompt lookup (the reference's demo/llama3/demo.py:760-770): the n-gram tasks produce the ids the embedding reads
            all_tokens = mpk.attach_input(self.meta["tokens"], "all_tokens")
            spec_tokens = mpk.draft_forward_layer_dispatcher(spec_decode_config=spec, tokens=all_tokens, grid_dim=(96, 1, 1), block_dim=(128, 1, 1))
            x = spec_tokens
            t["spec_tokens"] = spec_tokens
        cos = mpk.attach_input(self.cos, "cos_position_embedding")
        sin = mpk.attach_input(self.sin, "sin_position_embedding")
        new = lambda name, cols, dt=mi.bfloat16: mpk.new_tensor(dims=(B, cols), dtype=dt, name=name, io_category="cuda_tensor")
        y = new("embed_out", H)
        rmsnorm_out = new("rmsnorm_out", H)
        attn_in = new("attn_in", fused1)
        attn_out = new("attn_out", nq * D)
        q_ws = new("ck_fmha_q_workspace", nq * D)
        lse_acc = new("ck_fmha_lse_acc", nq, mi.float32)
        attn_proj_out = new("attn_proj_out", H)
        moe = s.num_experts > 0
        if moe:
            E, topk, MI = s.num_experts, s.num_experts_per_tok, s.moe_intermediate_size
            new3 = lambda name, cols: mpk.new_tensor(dims=(B, topk, cols), dtype=mi.bfloat16, name=name, io_category="cuda_tensor")
            moe_gate_out = new("moe_gate_out", E)
            moe_topk_weight = new("moe_topk_weight", topk, mi.float32)
            moe_routing_indices = mpk.new_tensor(dims=(E, B), dtype=mi.int32, name="moe_routing_indices", io_category="cuda_tensor")
            moe_mask = mpk.new_tensor(dims=(E + 1,), dtype=mi.int32, name="moe_mask", io_category="cuda_tensor")
            mlp_mid, silu_mul_out, mlp_out = new3("mlp_mid", 2 * MI), new3("silu_mul_out", MI), new3("mlp_out", H)
            mlp_weighted_sum_out = new("mlp_weighted_sum_out", H)
            t.update(moe_gate_out=moe_gate_out, moe_topk_weight=moe_topk_weight, moe_routing_indices=moe_routing_indices, moe_mask=moe_mask,
                     mlp_weighted_sum_out=mlp_weighted_sum_out)
        else:
            mlp_mid = new("mlp_mid", 2 * I)
            silu_mul_out = new("silu_mul_out", I)
            mlp_out = new("mlp_out", H)
        argmax_in = new("argmax_in", s.vocab_size)
        argmax_tasks = mpk.num_workers if s.vocab_size % mpk.num_workers == 0 else 1
        for cand in (240, 256, 128, 64, 32, 16, 8, 4, 2):
            if s.vocab_size % cand == 0:
                argmax_tasks = cand
                break
        argmax_part_value = new("argmax_part_value", argmax_tasks)
        argmax_part_index = new("argmax_part_index", argmax_tasks, mi.int64)
        argmax_out = mpk.attach_input(self.meta["output_tokens"], "output_token")
        t.update(embed_out=y, attn_in=attn_in, attn_out=attn_out, argmax_in=argmax_in, rmsnorm_out=rmsnorm_out, q_ws=q_ws,
                 attn_proj_out=attn_proj_out, silu_mul_out=silu_mul_out, mlp_out=mlp_out, mlp_mid=mlp_mid)
        wemb = mpk.attach_input(w["embed"], "embed_tokens")
        mpk.embed_layer(input=x, weight=wemb, output=y, grid_dim=(1, 1, 1), block_dim=(128, 1, 1), input_source=1)
        x = y
        tile_n = 64
        m_tiles = max(1, B // 16) if gang else 1
        if gang and B % m_tiles:
            m_tiles = 1

        def norm(inp, wn):
            if gang:
                mpk.gang_rmsnorm_layer(input=inp, weight=wn, output=rmsnorm_out)
            else:
                mpk.rmsnorm_layer(input=inp, weight=wn, output=rmsnorm_out, grid_dim=(B, 1, 1), block_dim=(128, 1, 1))

        for i, lw in enumerate(w["layers"]):
            proj_out, layer_out = attn_proj_out, mlp_out
            if self.tap_last_layer_input and i == len(w["layers"]) - 1:
                t["layer_in_tap"] = new("layer_in_tap", H)
                mpk.identity_layer(input=x, output=t["layer_in_tap"], grid_dim=(1, 1, 1), block_dim=(128, 1, 1))
            w_norm = mpk.attach_input(lw["input_norm"], f"layer_{i}_input_layernorm")
            w_q = mpk.attach_input(lw["q_proj"], f"layer_{i}_q_proj")
            w_k = mpk.attach_input(lw["k_proj"], f"layer_{i}_k_proj")
            w_v = mpk.attach_input(lw["v_proj"], f"layer_{i}_v_proj")
            w_qkv = mpk.shuffle_tensors(inputs=[w_q, w_k, w_v], shuffled_dim=0, num_groups=nkv, name=f"layer_{i}_qkv_proj")
            norm(x, w_norm)
            if gang:
                mpk.gang_linear_layer(input=rmsnorm_out, weight=w_qkv, output=attn_in, tile_n=tile_n, output_stride=w_qkv.dim(0), m_tiles=m_tiles)
            else:
                mpk.linear_layer(input=rmsnorm_out, weight=w_qkv, output=attn_in, grid_dim=(fused1 // 64, 1, 1), block_dim=(128, 1, 1))
            w_qn = mpk.attach_input(lw["q_norm"], f"layer_{i}_q_norm")
            w_kn = mpk.attach_input(lw["k_norm"], f"layer_{i}_k_norm")
            k_cache = mpk.attach_input(self.k_cache[i], f"layer_{i}_k_cache")
            v_cache = mpk.attach_input(self.v_cache[i], f"layer_{i}_v_cache")
            if gang:
                mpk.gang_paged_attention_split_kv_layer(
                    input=attn_in, k_cache=k_cache, v_cache=v_cache, q_norm=w_qn, k_norm=w_kn, cos_pos_embed=cos, sin_pos_embed=sin,
                    lse=lse_acc, output=attn_out, q_workspace=q_ws, attention_params=(nq, 1, nq * D), block_dim=(256, 1, 1))
            else:
                mpk.kv_cache_update_layer(input=attn_in, k_cache=k_cache, v_cache=v_cache, q_norm=w_qn, k_norm=w_kn, cos_pos_embed=cos,
                                          sin_pos_embed=sin, q_workspace=q_ws, grid_dim=(self.R, nkv, 1), block_dim=(256, 1, 1))
                mpk.paged_attention_ck_fmha_layer(q_workspace=q_ws, k_cache=k_cache, v_cache=v_cache, o_acc=attn_out, lse_acc=lse_acc,
                                                  attention_params=(nq, 1, self.R), grid_dim=(self.R, nkv, 1), block_dim=(256, 1, 1))
            w_o = mpk.attach_input(lw["o_proj"], f"layer_{i}_o_proj")
            if gang:
                mpk.gang_linear_with_residual_layer(input=attn_out, weight=w_o, residual=x, output=proj_out, tile_n=tile_n, output_stride=H, m_tiles=m_tiles)
            else:
                mpk.linear_with_residual_layer(input=attn_out, weight=w_o, residual=x, output=proj_out, grid_dim=(H // 64, 1, 1), block_dim=(256, 1, 1))
            x = proj_out
            w_norm2 = mpk.attach_input(lw["post_norm"], f"layer_{i}_post_attn_layernorm")
            if moe:
                # demo/qwen3/demo_30B_A3B.py:675-754
                w_router = mpk.attach_input(lw["router"], f"layer_{i}_moe_gate")
                w_gatedup = mpk.attach_input(lw["gate_up_proj"], f"layer_{i}_experts_gate_up_proj")
                w_down = mpk.attach_input(lw["down_proj"], f"layer_{i}_experts_down_proj")
                norm(x, w_norm2)
                mpk.linear_layer(input=rmsnorm_out, weight=w_router, output=moe_gate_out, grid_dim=(1, 1, 1), block_dim=(256, 1, 1))
                mpk.moe_topk_softmax_routing_layer(input=moe_gate_out, output=(moe_topk_weight, moe_routing_indices, moe_mask),
                                                   grid_dim=(1, 1, 1), block_dim=(256, 1, 1))
                if gang:
                    mpk.gang_moe_w13_linear_layer(input=rmsnorm_out, weight=w_gatedup, moe_routing_indices=moe_routing_indices,
                                                  moe_mask=moe_mask, output=mlp_mid)
                else:
                    mpk.moe_w13_linear_layer(input=rmsnorm_out, weight=w_gatedup, moe_routing_indices=moe_routing_indices, moe_mask=moe_mask,
                                             output=mlp_mid, grid_dim=(10, w_gatedup.dim(1) // 64, 1), block_dim=(256, 1, 1))
                mpk.moe_silu_mul_layer(input=mlp_mid, output=silu_mul_out, grid_dim=(B, topk, 1), block_dim=(256, 1, 1))
                if gang:
                    mpk.gang_moe_w2_linear_layer(input=silu_mul_out, weight=w_down, moe_routing_indices=moe_routing_indices, moe_mask=moe_mask,
                                                 output=mlp_out)
                else:
                    mpk.moe_w2_linear_layer(input=silu_mul_out, weight=w_down, moe_routing_indices=moe_routing_indices, moe_mask=moe_mask,
                                            output=mlp_out, grid_dim=(8, w_down.dim(1) // 64, 1), block_dim=(256, 1, 1))
                mpk.moe_mul_sum_add_layer(input=mlp_out, weight=moe_topk_weight, residual=x, output=mlp_weighted_sum_out,
                                          grid_dim=(B, max(1, H // 256), 1), block_dim=(256, 1, 1))
                x = mlp_weighted_sum_out
                continue
            w_gate = mpk.attach_input(lw["gate_proj"], f"layer_{i}_gate_proj")
            w_up = mpk.attach_input(lw["up_proj"], f"layer_{i}_up_proj")
            groups = (2 * I) // 256
            w_gu = mpk.shuffle_tensors(inputs=[w_gate, w_up], shuffled_dim=0, num_groups=groups, name=f"layer_{i}_gatedup_proj")
            norm(x, w_norm2)
            if gang:
                mpk.gang_linear_silu_layer(input=rmsnorm_out, weight=w_gu, output=silu_mul_out, tile_n=tile_n, output_stride=I, m_tiles=m_tiles)
            else:
                mpk.linear_layer(input=rmsnorm_out, weight=w_gu, output=mlp_mid, grid_dim=((2 * I) // 64, 1, 1), block_dim=(128, 1, 1))
                mpk.silu_mul_layer(input=mlp_mid, output=silu_mul_out, grid_dim=(groups, 1, 1), block_dim=(128, 1, 1))
            w_d = mpk.attach_input(lw["down_proj"], f"layer_{i}_down_proj")
            if gang:
                mpk.gang_linear_with_residual_layer(input=silu_mul_out, weight=w_d, residual=x, output=layer_out, tile_n=tile_n, output_stride=H, m_tiles=m_tiles)
            else:
                mpk.linear_with_residual_layer(input=silu_mul_out, weight=w_d, residual=x, output=layer_out, grid_dim=(H // 64, 1, 1), block_dim=(256, 1, 1))
            x = layer_out
        t["hidden_out"] = x
        if not self.with_head:
            return
        w_fn = mpk.attach_input(w["final_norm"], "model_norm_weight")
        w_lm = mpk.attach_input(w["lm_head"], "lm_head")
        norm(x, w_fn)
        mpk.linear_layer(input=rmsnorm_out, weight=w_lm, output=argmax_in, grid_dim=(argmax_tasks, 1, 1), block_dim=(128, 1, 1))
        mpk.argmax_partial_layer(input=argmax_in, output=(argmax_part_value, argmax_part_index), grid_dim=(argmax_tasks, 1, 1), block_dim=(128, 1, 1))
        mpk.argmax_reduce_layer(input=(argmax_part_value, argmax_part_index), output=argmax_out, grid_dim=(1, 1, 1), block_dim=(128, 1, 1))
        if spec_tokens is not None:
            t["verify_out"] = mpk.verify_layer_dispatcher(spec_decode_config=spec, spec_tokens=spec_tokens, target_output=argmax_out,
                                                          grid_dim=(1, 1, 1), block_dim=(128, 1, 1))

    # ------------------------------------------------------------------ running
    def load_prompts(self, prompts):
        """prompts: list of 1-D int64 tensors (one per request, at most total_requests)."""
        assert len(prompts) <= self.total_requests
        tokens = torch.zeros(self.total_requests, self.max_seq, dtype=torch.int64)
        plen = torch.zeros(self.total_requests, dtype=torch.int32)
        for r, p in enumerate(prompts):
            assert 0 < len(p) < self.max_seq
            tokens[r, :len(p)] = p.cpu()
            plen[r] = len(p)
        self.meta["tokens"].copy_(tokens)
        self.meta["prompt_lengths"].copy_(plen)
        torch.cuda.synchronize()
        self.mpk.init_request_resources()

    def generate(self, prompts, stream=None):
        """Run every request to max_seq_length-1 tokens (or EOS) in one persistent launch; returns (tokens, steps) on the CPU."""
        self.load_prompts(prompts)
        self.mpk(default_stream=stream)
        return self.meta["tokens"].cpu(), self.meta["step"].cpu()

    def logits(self):
        return self.t["argmax_in"].to_torch()


def main():
    ap = argparse.ArgumentParser(description="Qwen3-shaped random-init decode on the MI355X persistent megakernel")
    ap.add_argument("--max-num-batched-tokens", type=int, default=1)
    ap.add_argument("--max-num-batched-requests", type=int, default=None)
    ap.add_argument("--max-seq-length", type=int, default=1200)
    ap.add_argument("--max-new-tokens", type=int, default=1024)
    ap.add_argument("--prompt-length", type=int, default=80)
    ap.add_argument("--page-size", type=int, default=4096)
    ap.add_argument("--num-layers", type=int, default=36)
    ap.add_argument("--mode", choices=["fleet", "mpk"], default="fleet")
    ap.add_argument("--model", choices=["qwen3-8b", "qwen3-30b-a3b"], default="qwen3-8b")
    ap.add_argument("--spec-decode", choices=["promptlookup"], default=None,
                    help="prompt-lookup speculative decoding: a decoding request also runs the tokens that followed the earliest earlier "
                         "occurrence of its last --ngram-size tokens and keeps those the model agrees with")
    ap.add_argument("--ngram-size", type=int, default=3)
    ap.add_argument("--spec-length", type=int, default=5)
    args = ap.parse_args()
    shape = Qwen3Shape(num_layers=args.num_layers) if args.model == "qwen3-8b" else Qwen3Shape.qwen3_30b_a3b(min(args.num_layers, 48))
    B = args.max_num_batched_tokens
    R = args.max_num_batched_requests or B
    max_seq = min(args.max_seq_length, args.prompt_length + args.max_new_tokens + 1)
    w = random_weights(shape, 0)
    spec = mi.mpk.spec_decode_class(args.spec_decode, ngram_size=args.ngram_size, spec_length=args.spec_length)
    if spec is not None:
        B = max(B, R * (spec.spec_length + 1))
    dec = Qwen3Decoder(shape, w, B, R, max_seq, args.page_size, mode=args.mode, spec_decode_config=spec,
                       max_tokens_per_request=None if spec is None else max(8, spec.spec_length + 1))
    prompts = [torch.randint(0, shape.vocab_size, (args.prompt_length,), generator=torch.Generator().manual_seed(r)) for r in range(R)]
    dec.load_prompts(prompts)
    prefill_iters = math.ceil(args.prompt_length * R / B)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.mpk.run_steps(prefill_iters)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    done = dec.mpk.run_steps(1 << 30)
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    st = dec.mpk.stats()
    decode_iters = st["iterations"] - prefill_iters
    if spec is not None:
        new_tokens = int((dec.meta["step"].cpu() - args.prompt_length).clamp(min=0).sum())
        print(f"prompt lookup (n-gram {spec.ngram_size}, {spec.spec_length} guesses): {new_tokens} tokens in {st['iterations']} iterations "
              f"({new_tokens / max(1, decode_iters):.2f} per decode iteration), {new_tokens / max(1e-9, t2 - t1):.0f} tokens/s")
    print(f"prefill: {prefill_iters} iterations in {(t1 - t0) * 1e3:.1f} ms; decode: {decode_iters} iterations in {(t2 - t1) * 1e3:.1f} ms "
          f"({(t2 - t1) * 1e3 / max(1, decode_iters):.3f} ms/token at BS={R}); finished={done}")


if __name__ == "__main__":
    main()
