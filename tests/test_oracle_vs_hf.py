"""The oracle's model COMPOSITION (layer wiring, q/k-norm placement, RoPE convention, GQA head grouping, SwiGLU, residuals,
final norm + head) against an independent library: Hugging Face transformers' Qwen3ForCausalLM, which is what the
reference's modeling_qwen3.py derives from (demo/qwen3/models/modeling_qwen3.py:1-30) and what its MoE driver runs
(demo/qwen3/demo_30B_A3B.py:1).  CPU only; tiny random configurations; no files are loaded.

* dense: the oracle's float64 order equals the HF model evaluated in float64 to 1e-6 (same eps, unrounded RoPE tables),
  and the two bf16 orders the GPU tests use stay within bf16 tolerance of that float64 result -- so a dropped residual,
  a transposed projection, a wrong rotate-half sign or head grouping in any order fails here;
* mixture of experts: moe_block_t equals HF's sparse MoE block on the same bf16 inputs (same operator order), and the
  kernel-order moe_route_k / moe_mlp_k agree with it within bf16 tolerance.
The installed transformers (5.x) is newer than the reference's pin (4.57.1); the model definition is the same."""
import pytest
import torch

transformers = pytest.importorskip("transformers")

from oracle.qwen3_ref import KVCache, Qwen3Config, Qwen3Oracle, moe_block_t, moe_mlp_k, moe_route_k, moe_route_margin  # noqa: E402


def _oracle_weights(sd, n_layers, moe=False):
    w = {"embed": sd["model.embed_tokens.weight"], "final_norm": sd["model.norm.weight"], "lm_head": sd["lm_head.weight"], "layers": []}
    for i in range(n_layers):
        p = f"model.layers.{i}."
        lw = {"input_norm": sd[p + "input_layernorm.weight"], "q_proj": sd[p + "self_attn.q_proj.weight"], "k_proj": sd[p + "self_attn.k_proj.weight"],
              "v_proj": sd[p + "self_attn.v_proj.weight"], "q_norm": sd[p + "self_attn.q_norm.weight"], "k_norm": sd[p + "self_attn.k_norm.weight"],
              "o_proj": sd[p + "self_attn.o_proj.weight"], "post_norm": sd[p + "post_attention_layernorm.weight"]}
        if moe:
            lw.update(router=sd[p + "mlp.gate.weight"], gate_up_proj=sd[p + "mlp.experts.gate_up_proj"], down_proj=sd[p + "mlp.experts.down_proj"])
        else:
            lw.update(gate_proj=sd[p + "mlp.gate_proj.weight"], up_proj=sd[p + "mlp.up_proj.weight"], down_proj=sd[p + "mlp.down_proj.weight"])
        w["layers"].append(lw)
    return w


def test_dense_model_composition_matches_transformers():
    from transformers import Qwen3Config as HFConfig, Qwen3ForCausalLM
    torch.manual_seed(0)
    hc = HFConfig(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=3, num_attention_heads=8, num_key_value_heads=2, head_dim=128,
                  rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=64, tie_word_embeddings=False, attention_bias=False)
    hf = Qwen3ForCausalLM(hc).eval()
    with torch.no_grad():  # random norm weights: all-ones would hide a norm applied with the wrong weight
        for n, p in hf.named_parameters():
            if "norm" in n:
                p.copy_(1.0 + 0.1 * torch.randn_like(p))
        for p in hf.parameters():       # weights rounded to bf16, as the oracle holds them (buffers -- the rotary inverse
            p.copy_(p.to(torch.bfloat16).to(p.dtype))  # frequencies -- keep their precision)
    sd = {k: v.to(torch.bfloat16) for k, v in hf.state_dict().items()}
    cfg = Qwen3Config(hidden_size=256, num_q_heads=8, num_kv_heads=2, head_dim=128, intermediate_size=512, num_layers=3, vocab_size=512, max_positions=64)
    w = _oracle_weights(sd, 3)
    ids = torch.randint(0, 512, (11,), generator=torch.Generator().manual_seed(5))
    with torch.no_grad():
        ref = hf.double()(ids[None]).logits[0]   # float64 evaluation of the bf16-valued weights, causal over the 11 tokens
    # unrounded RoPE tables computed the way the library does (fp32 inverse frequencies and angles)
    inv = 1.0 / (1e6 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    ang = torch.arange(64, dtype=torch.float32)[:, None] * inv[None, :]
    emb = torch.cat((ang, ang), -1)
    o64 = Qwen3Oracle(cfg, w, "f64", rope=(emb.cos().double(), emb.sin().double()))
    c64 = KVCache(cfg, 16, torch.float64)
    got = torch.cat([o64.forward(ids[:7], c64, 0)] + [o64.forward(ids[p:p + 1], c64, p) for p in range(7, 11)])  # prefill 7, then 4 single steps
    torch.testing.assert_close(got, ref, atol=2e-6, rtol=1e-6)
    # the two bf16 orders against the same float64 yardstick (bf16 tables: the orders' own)
    base = Qwen3Oracle(cfg, w, "f64")
    cb = KVCache(cfg, 16, torch.float64)
    exact = base.forward(ids, cb, 0)
    for order, atol in (("kernel", 3e-2), ("torch", 6e-2)):
        o = Qwen3Oracle(cfg, w, order)
        lg = o.forward(ids, KVCache(cfg, 16), 0).double()
        torch.testing.assert_close(lg, exact, atol=atol, rtol=2e-2)
        assert (lg.argmax(-1) == exact.argmax(-1)).float().mean() >= 0.8


def test_moe_block_matches_transformers():
    from transformers import Qwen3MoeConfig, Qwen3MoeForCausalLM
    torch.manual_seed(1)
    hc = Qwen3MoeConfig(vocab_size=512, hidden_size=256, intermediate_size=512, moe_intermediate_size=64, num_experts=16, num_experts_per_tok=4,
                        norm_topk_prob=True, num_hidden_layers=1, num_attention_heads=8, num_key_value_heads=2, head_dim=128, rms_norm_eps=1e-6,
                        rope_theta=1e6, max_position_embeddings=64, tie_word_embeddings=False, decoder_sparse_step=1, mlp_only_layers=[])
    hf = Qwen3MoeForCausalLM(hc).to(torch.bfloat16).eval()
    with torch.no_grad():
        for n, p in hf.named_parameters():  # the library leaves the fused expert tensors at its default init: give them the usual scale
            if "experts" in n or "mlp.gate" in n:
                p.copy_((torch.randn(p.shape) * 0.05).to(p.dtype))
    blk = hf.model.layers[0].mlp
    sd = hf.state_dict()
    router, gate_up, down = sd["model.layers.0.mlp.gate.weight"], sd["model.layers.0.mlp.experts.gate_up_proj"], sd["model.layers.0.mlp.experts.down_proj"]
    h = torch.randn(9, 256, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    with torch.no_grad():
        out = blk(h[None])
    ref = (out[0] if isinstance(out, tuple) else out).reshape(9, 256)
    got = moe_block_t(h, router, gate_up, down, 4)
    torch.testing.assert_close(got.float(), ref.float(), atol=4e-3, rtol=1.6e-2)   # same operator order: at most a bf16 rounding apart
    # kernel order (fp32 router weights, per-slot rounding): within bf16 tolerance of the library block where routing is not a near-tie
    logits = (h.float() @ router.float().t()).to(torch.bfloat16)
    ok = moe_route_margin(logits, 4) > 0.02
    wts, exp = moe_route_k(logits, 4)
    k_out = moe_mlp_k(h, torch.zeros_like(h), gate_up, down, wts, exp)[0]
    assert int(ok.sum()) >= 6
    torch.testing.assert_close(k_out[ok].float(), ref[ok].float(), atol=2e-2, rtol=3e-2)
