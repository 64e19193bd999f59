"""Mixture-of-experts decode path (Qwen3-30B-A3B shape): router softmax/top-k, per-expert W13 + SwiGLU, per-expert W2,
weighted sum + residual -- through the PersistentKernel MoE layers (reference: demo/qwen3/demo_30B_A3B.py:675-754,
python/mirage/mpk/persistent_kernel.py:1203-1436), compared stage by stage with the CPU oracle on the GPU's own
stage inputs, then end to end through the greedy loop.

Closest reference checks: tests/runtime_python/test_moe_linear.py:33-73 (routing/mask construction, assert_close
rtol=atol=1e-2), tests/runtime_python/blackwell/sm100_moe/test_gate_topk.py:37-83 (softmax -> top-k -> renormalise)."""
import functools

import pytest
import torch

from helpers import bf16_ulp_diff, make_meta, make_mpk

pytestmark = pytest.mark.gpu


@functools.lru_cache(maxsize=2)
def _moe_inputs(H, E, MI, B, seed):
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    return {
        "x": torch.randn(B, H, generator=g).to(bf),
        "nw": (1.0 + 0.02 * torch.randn(H, generator=g)).to(bf),
        "router": (0.02 * torch.randn(E, H, generator=g)).to(bf),
        "w13": (0.02 * torch.randn(E, 2 * MI, H, generator=g)).to(bf),
        "w2": (0.02 * torch.randn(E, H, MI, generator=g)).to(bf),
    }


def _build_block(mpk, d, B, E, topk, MI, H, gang):
    import mirage as mi
    t = {k: mpk.attach_input(v, k) for k, v in d.items()}
    n = mpk.new_tensor((B, H), name="n")
    gate = mpk.new_tensor((B, E), name="gate")
    tw = mpk.new_tensor((B, topk), dtype=mi.float32, name="topk_w")
    ri = mpk.new_tensor((E, B), dtype=mi.int32, name="routing")
    mask = mpk.new_tensor((E + 1,), dtype=mi.int32, name="mask")
    mid, act, y = mpk.new_tensor((B, topk, 2 * MI), name="mid"), mpk.new_tensor((B, topk, MI), name="act"), mpk.new_tensor((B, topk, H), name="y")
    out = mpk.new_tensor((B, H), name="out")
    mpk.rmsnorm_layer(input=t["x"], weight=t["nw"], output=n, grid_dim=(B, 1, 1), block_dim=(128, 1, 1))
    mpk.linear_layer(input=n, weight=t["router"], output=gate, grid_dim=(1, 1, 1), block_dim=(256, 1, 1))
    mpk.moe_topk_softmax_routing_layer(input=gate, output=(tw, ri, mask), grid_dim=(1, 1, 1), block_dim=(256, 1, 1))
    if gang:
        mpk.gang_moe_w13_linear_layer(input=n, weight=t["w13"], moe_routing_indices=ri, moe_mask=mask, output=mid)
        mpk.moe_silu_mul_layer(input=mid, output=act, grid_dim=(B, topk, 1), block_dim=(256, 1, 1))
        mpk.gang_moe_w2_linear_layer(input=act, weight=t["w2"], moe_routing_indices=ri, moe_mask=mask, output=y)
    else:
        mpk.moe_w13_linear_layer(input=n, weight=t["w13"], moe_routing_indices=ri, moe_mask=mask, output=mid, grid_dim=(10, 2 * MI // 64, 1),
                                 block_dim=(256, 1, 1))
        mpk.moe_silu_mul_layer(input=mid, output=act, grid_dim=(B, topk, 1), block_dim=(256, 1, 1))
        mpk.moe_w2_linear_layer(input=act, weight=t["w2"], moe_routing_indices=ri, moe_mask=mask, output=y, grid_dim=(8, H // 64, 1), block_dim=(256, 1, 1))
    mpk.moe_mul_sum_add_layer(input=y, weight=tw, residual=t["x"], output=out, grid_dim=(B, max(1, H // 256), 1), block_dim=(256, 1, 1))
    return dict(n=n, gate=gate, tw=tw, ri=ri, mask=mask, mid=mid, act=act, y=y, out=out)


def _close(name, a, b, max_ulp=1.0, max_flip=0.05, floor=1e-3):
    ulp, _ = bf16_ulp_diff(a, b, floor=floor)
    flips = float((a.float() != b.float()).float().mean())
    assert ulp <= max_ulp, f"{name}: differs from the oracle by {ulp} bf16 ulp"
    assert flips < max_flip, f"{name}: {flips:.1%} of the values differ from the oracle"


@pytest.mark.parametrize("gang", [False, True])
@pytest.mark.parametrize("H,E,topk,MI,B,M", [
    (2048, 128, 8, 768, 1, 1),    # Qwen3-30B-A3B layer shape, single token (routing, SwiGLU and combine folded into the linears)
    (2048, 128, 8, 768, 8, 8),    # same shape, batched: top-k / combine stages
    (2048, 128, 8, 768, 8, 3),    # fewer tokens than batch rows
    (512, 16, 4, 128, 4, 4),      # expert count and k below one wavefront's width
    (1024, 40, 6, 384, 2, 1),     # expert count not a multiple of 64, k with a ragged last segment
    (1024, 40, 6, 384, 64, 64),   # maximum batch
])
def test_moe_block_stagewise(gang, H, E, topk, MI, B, M):
    from oracle.qwen3_ref import linear_k, moe_mlp_k, moe_route_k, moe_routing_tables, rmsnorm_k
    d = _moe_inputs(H, E, MI, B, H + E)
    dg = {k: v.cuda() for k, v in d.items()}
    meta = make_meta(B, 64, B, B, B)
    mpk = make_mpk(meta, 64, B, B, B, 64, mode="onepass")
    t = _build_block(mpk, dg, B, E, topk, MI, H, gang)
    mpk.compile()
    mpk.run_once(list(range(M)), [0] * M)
    g = {k: v.to_torch().cpu() for k, v in t.items()}
    x = d["x"][:M]
    # norm and router logits
    n_ref = rmsnorm_k(x, d["nw"])
    _close("rmsnorm", g["n"][:M], n_ref)
    gate_ref = linear_k(g["n"][:M], d["router"])
    _close("router logits", g["gate"][:M], gate_ref)
    # routing from the GPU's own logits: integer outputs exact, fp32 weights to rounding of the sums
    w_ref, e_ref = moe_route_k(g["gate"][:M], topk)
    routing_ref, active_ref = moe_routing_tables(e_ref, E)
    # ties between bf16 logits are common (128 experts, 8-bit mantissa): the tie rule (lower expert id) is part of the check
    assert torch.equal(g["ri"][:, :M], routing_ref), "routing table differs from the oracle"
    torch.testing.assert_close(g["tw"][:M], w_ref, rtol=2e-6, atol=1e-9)
    n_act = int(g["mask"][E])
    assert n_act == len(active_ref) and sorted(g["mask"][:n_act].tolist()) == active_ref
    assert torch.allclose(g["tw"][:M].sum(-1), torch.ones(M), atol=1e-6)
    # expert MLP on the GPU's normalised rows and routing
    out_ref, mid_ref, act_ref, y_ref = moe_mlp_k(g["n"][:M], x, d["w13"], d["w2"], g["tw"][:M], e_ref)
    _close("W13 output", g["mid"][:M], mid_ref)
    # SwiGLU and W2 from the GPU's own inputs (bit-exact up to expf / accumulation order)
    from oracle.qwen3_ref import silu_mul_k
    _close("SwiGLU", g["act"][:M], silu_mul_k(g["mid"][:M, :, :MI], g["mid"][:M, :, MI:]), max_flip=0.01)
    y_own = torch.stack([torch.stack([linear_k(g["act"][tk, s][None], d["w2"][int(e_ref[tk, s])])[0] for s in range(topk)]) for tk in range(M)])
    _close("W2 output", g["y"][:M], y_own)
    acc = x.float()
    for s in range(topk):
        acc = acc + g["y"][:M, s].float() * g["tw"][:M, s, None]
    _close("combine", g["out"][:M], acc.to(torch.bfloat16), max_flip=0.01)
    # end to end against the oracle chain: north-star tolerance
    torch.testing.assert_close(g["out"][:M].float(), out_ref.float(), atol=2e-2, rtol=1e-2)
    st = mpk.stats()
    assert st["aborted"] == 0
    mpk.finalize()


def test_moe_standalone_stages_and_user_routing():
    """The activation and combine tasks on their own (not behind a per-expert linear) and a W2-type linear driven by a
    caller-written routing table, as tests/runtime_python/test_moe_linear.py:33-61 builds one."""
    import mirage as mi
    from oracle.qwen3_ref import linear_k, silu_mul_k
    B, E, topk, MI, H = 5, 12, 3, 192, 256
    g = torch.Generator().manual_seed(5)
    bf = torch.bfloat16
    mid = torch.randn(B, topk, 2 * MI, generator=g).to(bf)
    yin = torch.randn(B, topk, H, generator=g).to(bf)
    tw = torch.rand(B, topk, generator=g)
    res = torch.randn(B, H, generator=g).to(bf)
    xin = torch.randn(B, topk, MI, generator=g).to(bf)
    w2 = (0.05 * torch.randn(E, H, MI, generator=g)).to(bf)
    experts = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(B)])
    routing = torch.zeros(E, B, dtype=torch.int32)
    for tk in range(B):
        for s in range(topk):
            routing[experts[tk, s], tk] = s + 1
    dev = {k: v.cuda() for k, v in dict(mid=mid, yin=yin, tw=tw, res=res, xin=xin, w2=w2, routing=routing).items()}
    dev["mask"] = torch.zeros(E + 1, dtype=torch.int32, device="cuda")
    meta = make_meta(B, 64, B, B, B)
    mpk = make_mpk(meta, 64, B, B, B, 64, mode="onepass")
    t = {k: mpk.attach_input(v, k) for k, v in dev.items()}
    act = mpk.new_tensor((B, topk, MI), name="act")
    out = mpk.new_tensor((B, H), name="out")
    y2 = mpk.new_tensor((B, topk, H), name="y2")
    mpk.moe_silu_mul_layer(input=t["mid"], output=act, grid_dim=(B, topk, 1), block_dim=(256, 1, 1))
    mpk.moe_mul_sum_add_layer(input=t["yin"], weight=t["tw"], residual=t["res"], output=out, grid_dim=(B, 1, 1), block_dim=(256, 1, 1))
    mpk.moe_w2_linear_layer(input=t["xin"], weight=t["w2"], moe_routing_indices=t["routing"], moe_mask=t["mask"], output=y2, grid_dim=(8, H // 64, 1),
                            block_dim=(256, 1, 1))
    kinds = [l.split()[1] for l in mpk.describe_program().splitlines()]
    assert kinds == ["SILU_MUL(moe)", "MOE_COMBINE", "MOE_LINEAR"]
    mpk.compile()
    for M in (B, 1, 2):
        act.to_torch().zero_(), out.to_torch().zero_(), y2.to_torch().zero_()
        torch.cuda.synchronize()
        mpk.run_once(list(range(M)), [0] * M)
        _close("standalone SwiGLU", act.to_torch()[:M].cpu(), silu_mul_k(mid[:M, :, :MI], mid[:M, :, MI:]), max_flip=0.01)
        acc = res[:M].float()
        for s in range(topk):
            acc = acc + yin[:M, s].float() * tw[:M, s, None]
        _close("standalone combine", out.to_torch()[:M].cpu(), acc.to(bf), max_flip=0.01)
        y_ref = torch.stack([torch.stack([linear_k(xin[tk, s][None], w2[int(experts[tk, s])])[0] for s in range(topk)]) for tk in range(M)])
        _close("W2 with caller routing", y2.to_torch()[:M].cpu(), y_ref)
        mask = dev["mask"].cpu()
        act_ref = sorted(set(experts[:M].flatten().tolist()))
        assert int(mask[E]) == len(act_ref) and sorted(mask[:len(act_ref)].tolist()) == act_ref
        # rows of tokens outside the iteration stay untouched
        assert float(act.to_torch()[M:].float().abs().sum()) == 0 and float(y2.to_torch()[M:].float().abs().sum()) == 0
    mpk.finalize()


def _moe_cfg(layers=2, vocab=2048):
    from oracle.qwen3_ref import Qwen3Config
    return Qwen3Config(hidden_size=1024, num_q_heads=8, num_kv_heads=2, head_dim=128, intermediate_size=0, num_layers=layers, vocab_size=vocab,
                       num_experts=32, num_experts_per_tok=4, moe_intermediate_size=256)


def _decoder(cfg, w, **kw):
    from demo_qwen3 import Qwen3Decoder, Qwen3Shape
    from oracle.qwen3_ref import rope_tables
    shape = Qwen3Shape(cfg.hidden_size, cfg.num_q_heads, cfg.num_kv_heads, cfg.head_dim, cfg.intermediate_size, cfg.num_layers, cfg.vocab_size,
                       cfg.rope_theta, cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size)
    cos, sin = rope_tables(cfg, max(kw.get("max_seq_length", 1200), 16))
    wg = {"embed": w["embed"].cuda(), "layers": [{k: v.cuda() for k, v in lw.items()} for lw in w["layers"]],
          "final_norm": w["final_norm"].cuda(), "lm_head": w["lm_head"].cuda()}
    return Qwen3Decoder(shape, wg, cos_sin=(cos.cuda(), sin.cuda()), **kw)


@pytest.mark.parametrize("mode", ["fleet", "mpk"])
def test_moe_bs1_greedy_matches_oracle_teacher_forced(mode):
    """BS=1 greedy decode of a small mixture-of-experts model: at every step the oracle (teacher-forced with the GPU's tokens)
    must agree on the logits within the north-star tolerance and on the argmax wherever its top-2 margin exceeds 0.05."""
    from oracle.qwen3_ref import KVCache, Qwen3Oracle, argmax_k, make_model_weights, make_prompt
    cfg = _moe_cfg()
    w = make_model_weights(cfg, seed=11)
    P, NEW = 10, 20
    max_seq = P + NEW + 1
    prompt = make_prompt(cfg, P, 2)
    dec = _decoder(cfg, w, max_num_batched_tokens=1, max_seq_length=max_seq, page_size=16, mode=mode)
    dec.load_prompts([prompt])
    orc = Qwen3Oracle(cfg, w, "kernel")
    cache = KVCache(cfg, max_seq)
    toks = prompt.tolist()
    n_margin = n_compared = 0
    for it in range(P + NEW - 1):
        dec.mpk.run_steps(1)
        gpu_logits = dec.logits()[0].float().cpu()
        gpu_tok = int(dec.meta["output_tokens"][0, 0].item())
        ref_logits = orc.forward(torch.tensor([toks[it]]), cache, it)[0].float()
        # top-k routing is discontinuous: a step where some layer's k-th and (k+1)-th router probabilities are within 1% of each
        # other (a bf16 rounding of the logits) may legitimately pick another expert; such steps are not compared
        if min(orc.route_margins) > 0.01:
            torch.testing.assert_close(gpu_logits, ref_logits, atol=2e-2, rtol=1e-2)
            n_compared += 1
            top2 = ref_logits.topk(2).values
            if float(top2[0] - top2[1]) > 0.05:
                assert gpu_tok == int(argmax_k(ref_logits[None].to(torch.bfloat16))[0]), f"argmax mismatch at iteration {it}"
                n_margin += 1
        if it + 1 >= P:
            toks.append(gpu_tok)
    assert n_margin > 0 and n_compared >= (P + NEW - 1) // 2
    assert dec.mpk.run_steps(4)
    assert dec.meta["tokens"][0].cpu().tolist()[:P + NEW] == toks[:P + NEW]
    dec.mpk.finalize()


@pytest.mark.parametrize("B,R_total", [(4, 6), (32, 40)])
def test_moe_batched_decode_continuous_batching(B, R_total):
    """BS=4 with six / BS=32 with forty requests of different prompt lengths (chunked prompt ingestion, slot reuse): every
    generated token must be the oracle's argmax wherever the oracle's margin exceeds 0.05."""
    from oracle.qwen3_ref import KVCache, Qwen3Oracle, argmax_k, make_model_weights, make_prompt
    cfg = _moe_cfg()
    w = make_model_weights(cfg, seed=12)
    max_seq = 30
    prompts = [make_prompt(cfg, 3 + (4 * r) % 11, 50 + r) for r in range(R_total)]
    dec = _decoder(cfg, w, max_num_batched_tokens=B, max_num_batched_requests=B, max_seq_length=max_seq, page_size=16, total_requests=R_total)
    toks, steps = dec.generate(prompts)
    assert all(int(s_) == max_seq - 1 for s_ in steps)
    orc = Qwen3Oracle(cfg, w, "kernel")
    hits = 0
    for r, prompt in enumerate(prompts):
        P = len(prompt)
        tk = toks[r].tolist()
        assert tk[:P] == prompt.tolist()
        cache = KVCache(cfg, max_seq + 1)
        lg = orc.forward(torch.tensor(tk[:P]), cache, 0)[-1:]
        for p in range(P, max_seq):
            top2 = lg[0].float().topk(2).values
            if float(top2[0] - top2[1]) > 0.05 and min(orc.route_margins) > 0.01:
                assert tk[p] == int(argmax_k(lg)[0]), f"request {r}: token at position {p} differs from the oracle"
                hits += 1
            if p + 1 < max_seq:
                lg = orc.forward(torch.tensor([tk[p]]), cache, p)
    assert hits >= 5 * (R_total // 6)
    assert dec.mpk.stats()["aborted"] == 0
    dec.mpk.finalize()
