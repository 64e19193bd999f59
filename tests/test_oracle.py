"""Pins the CPU oracle (oracle/qwen3_ref.py) against what the mathematics fixes: closed forms, float64 brute force on
small shapes, invariants and special cases -- chosen so a dropped term, a wrong sign/index or a transposed operand fails.
The reference holds no golden vectors for this path (its MI300 kernels have no tests; tests/runtime_python is CUDA-only
and mostly prints ratios), so these are the pins; the torch formulas mirrored are cited per test."""
import math

import numpy as np
import pytest
import torch

from oracle.qwen3_ref import (Qwen3Config, Qwen3Oracle, KVCache, argmax_k, attention_k, head_norm_rope_k, linear_k, linear_silu_k,
                              make_model_weights, make_prompt, rmsnorm_k, rmsnorm_t, rope_t, rope_tables, silu_mul_k)

BF = torch.bfloat16


def _bf(x):
    return x.to(BF)


def _ulp_close(a, b, n=1.0, floor=1e-3):
    af, bf = a.double(), b.double()
    scale = torch.maximum(af.abs(), bf.abs()).clamp_min(floor)
    ulp = torch.exp2(torch.floor(torch.log2(scale)) - 7)
    assert float(((af - bf).abs() / ulp).max()) <= n


def test_rmsnorm_closed_form_and_invariants():
    # formula: tests/runtime_python/test_rmsnorm.py:49-55 (x * rsqrt(mean(x^2)+eps) * w)
    g = torch.Generator().manual_seed(0)
    x = _bf(torch.randn(3, 256, generator=g))
    w = _bf(1 + 0.1 * torch.randn(256, generator=g))
    y = rmsnorm_k(x, w)
    xd, wd = x.double().numpy(), w.double().numpy()
    ref = xd / np.sqrt((xd ** 2).mean(-1, keepdims=True) + 1e-6) * wd
    _ulp_close(y, torch.from_numpy(ref))
    # scale invariance (power of two keeps bf16 exact): norm(4x) == norm(x) up to eps
    _ulp_close(rmsnorm_k(_bf(x.float() * 4), w), y)
    # unit weights: output rms is 1
    y1 = rmsnorm_k(x, torch.ones(256, dtype=BF)).float()
    assert torch.allclose(y1.pow(2).mean(-1).sqrt(), torch.ones(3), atol=5e-3)
    # a row of constant c normalises to sign(c) * w
    c = _bf(torch.full((1, 256), -3.0))
    _ulp_close(rmsnorm_k(c, w), -w[None])
    # torch-order variant: no eps, every op rounds to bf16 (modeling_qwen3.py:49-54) -- within a few bf16 ulp of the exact one
    _ulp_close(rmsnorm_t(x, w), torch.from_numpy(ref), n=4.0)


def test_linear_brute_force_and_special_cases():
    # CPU triple loop of the reference: tests/standalone/test_kernels.cpp:120-139 (C[m,n] = sum_k A[m,k] W[n,k])
    g = torch.Generator().manual_seed(1)
    x, W, r = _bf(torch.randn(2, 24, generator=g)), _bf(torch.randn(5, 24, generator=g)), _bf(torch.randn(2, 5, generator=g))
    ref = torch.zeros(2, 5, dtype=torch.float64)
    for m in range(2):
        for n in range(5):
            for k in range(24):
                ref[m, n] += float(x[m, k]) * float(W[n, k])
    _ulp_close(linear_k(x, W), ref)
    _ulp_close(linear_k(x, W, res=r), ref + r.double())
    # identity weight returns the input; one-hot input selects a weight column (catches a transposed operand)
    xi = _bf(torch.randn(3, 16, generator=g))
    assert torch.equal(linear_k(xi, torch.eye(16, dtype=BF)), xi)
    Wn = _bf(torch.randn(7, 16, generator=g))
    e3 = torch.zeros(1, 16, dtype=BF)
    e3[0, 3] = 1
    assert torch.equal(linear_k(e3, Wn)[0], Wn[:, 3])


def test_swiglu_closed_form():
    # formula: tests/runtime_python/test_silu_mul_linear.py:22-28 (silu(gate) * up)
    g = torch.Generator().manual_seed(2)
    gate, up = _bf(torch.randn(4, 64, generator=g) * 3), _bf(torch.randn(4, 64, generator=g))
    gd, ud = gate.double(), up.double()
    _ulp_close(silu_mul_k(gate, up), gd / (1 + torch.exp(-gd)) * ud)
    assert torch.equal(silu_mul_k(torch.zeros(1, 8, dtype=BF), up[:1, :8]), torch.zeros(1, 8, dtype=BF))
    # fused variant == unfused on exactly representable accumulators (single-term dot products)
    x = torch.zeros(1, 8, dtype=BF)
    x[0, 0] = 1
    Wg, Wu = _bf(torch.randn(6, 8, generator=g)), _bf(torch.randn(6, 8, generator=g))
    assert torch.equal(linear_silu_k(x, Wg, Wu), silu_mul_k(Wg[:, 0][None], Wu[:, 0][None]))
    # large negative gate -> 0, large positive gate -> gate*up
    big = _bf(torch.tensor([[-40.0, 40.0]]))
    out = silu_mul_k(big, _bf(torch.tensor([[2.0, 2.0]]))).float()
    assert abs(float(out[0, 0])) < 1e-12 and out[0, 1] == 80


def test_rope_is_a_complex_rotation():
    # reference formula: tests/runtime_python/test_multitoken_paged_attention.py:21-38; rope.py:79-80
    cfg = Qwen3Config()
    cos, sin = rope_tables(cfg, 64)
    # table: both halves equal, cos^2+sin^2 = 1 up to bf16, position 0 is the identity
    assert torch.equal(cos[:, :64], cos[:, 64:]) and torch.equal(sin[:, :64], sin[:, 64:])
    assert torch.all(cos[0] == 1) and torch.all(sin[0] == 0)
    assert torch.allclose(cos.float() ** 2 + sin.float() ** 2, torch.ones(64, 128), atol=2e-2)
    # frequencies: theta^(-2i/D); position 1, pair 0 rotates by exactly 1 radian
    assert abs(float(cos[1, 0]) - math.cos(1.0)) < 4e-3 and abs(float(sin[1, 0]) - math.sin(1.0)) < 4e-3
    assert abs(float(sin[7, 63]) - math.sin(7 * 1e6 ** (-126 / 128))) < 1e-5 + 4e-3 * abs(math.sin(7 * 1e6 ** (-126 / 128)))
    g = torch.Generator().manual_seed(3)
    x = _bf(torch.randn(5, 128, generator=g))
    pos = torch.tensor([0, 1, 7, 33, 63])
    y = head_norm_rope_k(x, None, cos[pos], sin[pos], qk_norm=False, rope=True)
    z = torch.complex(x.double()[:, :64], x.double()[:, 64:]) * torch.complex(cos[pos].double()[:, :64], sin[pos].double()[:, :64])
    _ulp_close(y, torch.cat((z.real, z.imag), -1))
    assert torch.equal(y[0], x[0])  # position 0
    # norm of each (i, i+64) pair is preserved up to table rounding
    n_in = (x.float()[:, :64] ** 2 + x.float()[:, 64:] ** 2).sqrt()
    n_out = (y.float()[:, :64] ** 2 + y.float()[:, 64:] ** 2).sqrt()
    assert torch.allclose(n_in, n_out, rtol=2e-2, atol=2e-2)
    # torch-order rope agrees within bf16 rounding of its intermediate products
    _ulp_close(rope_t(x, cos[pos], sin[pos]), torch.cat((z.real, z.imag), -1), n=3.0, floor=0.25)


def test_qk_norm_then_rope_rounds_between():
    cfg = Qwen3Config()
    cos, sin = rope_tables(cfg, 16)
    g = torch.Generator().manual_seed(4)
    x, w = _bf(torch.randn(2, 3, 128, generator=g)), _bf(1 + 0.1 * torch.randn(128, generator=g))
    pos = torch.tensor([5, 9])
    y = head_norm_rope_k(x, w, cos[pos][:, None], sin[pos][:, None])
    xn = rmsnorm_k(x, w)  # per-head norm over D=128, rounded to bf16 before the rotation
    y2 = head_norm_rope_k(xn, None, cos[pos][:, None], sin[pos][:, None], qk_norm=False)
    assert torch.equal(y, y2)


def test_attention_special_cases_and_brute_force():
    # reference formula: tests/runtime_python/test_multitoken_paged_attention.py:52-127 (softmax(QK^T/sqrt(D)) V, GQA)
    g = torch.Generator().manual_seed(5)
    nq, nkv, D, L = 8, 2, 128, 37
    q, K, V = _bf(torch.randn(nq, D, generator=g)), _bf(torch.randn(L, nkv, D, generator=g)), _bf(torch.randn(L, nkv, D, generator=g))
    out = attention_k(q, K, V)
    ref = torch.zeros(nq, D, dtype=torch.float64)
    for h in range(nq):
        kvh = h // (nq // nkv)  # q heads h*4..h*4+3 share kv head h (GQA grouping)
        s = (K[:, kvh].double() @ q[h].double()) / math.sqrt(D)
        p = torch.softmax(s, 0)
        ref[h] = p @ V[:, kvh].double()
    _ulp_close(out, ref, floor=1e-2)
    # L = 1: output is V[0] of the head's kv group
    o1 = attention_k(q, K[:1], V[:1])
    for h in range(nq):
        assert torch.equal(o1[h], V[0, h // 4])
    # constant K: uniform weights -> mean of V
    Kc = K[:1].expand(L, nkv, D).contiguous()
    _ulp_close(attention_k(q, Kc, V), V.double().mean(0).repeat_interleave(4, 0), floor=1e-2)
    # permutation invariance over cached positions
    perm = torch.randperm(L, generator=g)
    _ulp_close(attention_k(q, K[perm], V[perm]), out.double(), floor=1e-2)
    # split-KV merge associativity (merge rule: tasks/ampere/merge_splitkv.cuh:191-219)
    def part(lo, hi):
        s = torch.einsum("hd,lhd->hl", q.double(), K[lo:hi].double().repeat_interleave(4, 1)) / math.sqrt(D)
        m = s.max(-1).values
        p = torch.exp(s - m[:, None])
        return m, p.sum(-1), torch.einsum("hl,lhd->hd", p, V[lo:hi].double().repeat_interleave(4, 1))
    (m1, l1, o1_), (m2, l2, o2_) = part(0, 20), part(20, L)
    M = torch.maximum(m1, m2)
    merged = (o1_ * torch.exp(m1 - M)[:, None] + o2_ * torch.exp(m2 - M)[:, None]) / (l1 * torch.exp(m1 - M) + l2 * torch.exp(m2 - M))[:, None]
    _ulp_close(out, merged, floor=1e-2)


def test_argmax_planted_and_ties():
    # reference check: tests/runtime_python/test_argmax.py:18-36 (planted maximum at a random index)
    g = torch.Generator().manual_seed(6)
    x = _bf(torch.randn(3, 1000, generator=g))
    idx = torch.tensor([17, 999, 0])
    for r in range(3):
        x[r, idx[r]] = 65504.0
    assert torch.equal(argmax_k(x), idx)
    t = torch.zeros(2, 50, dtype=BF)
    t[0, 7] = t[0, 30] = 2.0   # tie -> lowest index
    t[1, :] = -1.0
    assert argmax_k(t).tolist() == [7, 0]


def test_model_orders_agree_and_prefill_equals_stepwise():
    """kernel-order and torch-order restatements differ only in rounding points: on a small model their logits agree
    within the north-star tolerance, and multi-token prefill equals token-by-token ingestion (causality)."""
    cfg = Qwen3Config(hidden_size=256, num_q_heads=8, num_kv_heads=2, head_dim=128, intermediate_size=512, num_layers=2, vocab_size=512)
    w = make_model_weights(cfg, 0)
    prompt = make_prompt(cfg, 7, 0)
    ok, ot = Qwen3Oracle(cfg, w, "kernel"), Qwen3Oracle(cfg, w, "torch")
    ck, ct = KVCache(cfg, 16), KVCache(cfg, 16)
    lk, lt = ok.forward(prompt, ck, 0), ot.forward(prompt, ct, 0)
    torch.testing.assert_close(lk.float(), lt.float(), atol=2e-2, rtol=1e-2)
    c2 = KVCache(cfg, 16)
    rows = [ok.forward(prompt[p:p + 1], c2, p)[0] for p in range(7)]

    def same(a, b):  # torch's gemm and gemv kernels sum in different orders: allow isolated bf16 flips
        torch.testing.assert_close(a.float(), b.float(), atol=1.6e-2, rtol=8e-3)
        assert float((a.float() != b.float()).float().mean()) < 0.05
    same(torch.stack(rows), lk)
    same(c2.k[:, :7], ck.k[:, :7])
    same(c2.v[:, :7], ck.v[:, :7])
    # chunked prefill (3 + 4 tokens) equals the single pass as well
    c3 = KVCache(cfg, 16)
    a = ok.forward(prompt[:3], c3, 0)
    b = ok.forward(prompt[3:], c3, 3)
    same(torch.cat((a, b)), lk)
    # causality: logits of the first 3 positions do not depend on later tokens
    c4 = KVCache(cfg, 16)
    other = prompt.clone()
    other[3:] = (other[3:] + 1) % cfg.vocab_size
    same(ok.forward(other, c4, 0)[:3], lk[:3])


def test_moe_router_matches_float64_topk_and_tie_rule():
    """moe_route_k against an independent float64 softmax + torch.topk + renormalise (the routing
    tests/runtime_python/blackwell/sm100_moe/test_gate_topk.py:37-52 uses as its reference), plus what the closed form
    fixes: weights sum to 1, planted probabilities come back, equal logits go to the lower expert id."""
    from oracle.qwen3_ref import moe_route_k, moe_routing_tables
    g = torch.Generator().manual_seed(0)
    T, E, k = 16, 128, 8
    # distinct logits so that top-k is unambiguous
    logits = (torch.randperm(T * E, generator=g).view(T, E).float() / (T * E) * 8 - 4).to(torch.bfloat16)
    logits = torch.stack([torch.unique(r)[torch.randperm(len(torch.unique(r)), generator=g)][:96] for r in logits])  # dedupe after bf16 rounding
    E = logits.shape[1]
    w, e = moe_route_k(logits, k)
    p64 = torch.softmax(logits.double(), -1)
    tv, ti = torch.topk(p64, k, dim=-1)
    assert torch.equal(e, ti), "selected experts (in slot order = descending probability) differ from float64 top-k"
    torch.testing.assert_close(w.double(), tv / tv.sum(-1, keepdim=True), rtol=1e-5, atol=0)
    torch.testing.assert_close(w.sum(-1), torch.ones(T), rtol=1e-6, atol=0)
    # planted probabilities: logits = log(p) for a known distribution -> weights = p_topk / sum(p_topk)
    p = torch.tensor([[0.4, 0.05, 0.3, 0.05, 0.2]])
    w2, e2 = moe_route_k(torch.log(p).to(torch.bfloat16), 2)
    assert e2.tolist() == [[0, 2]]
    torch.testing.assert_close(w2, torch.tensor([[0.4 / 0.7, 0.3 / 0.7]]), rtol=2e-2, atol=0)  # bf16 logits
    # ties: all-equal logits select experts 0..k-1 in order with weight 1/k (moe_topk_softmax_mi300.cuh:152-176)
    w3, e3 = moe_route_k(torch.zeros(2, 10, dtype=torch.bfloat16), 3)
    assert e3.tolist() == [[0, 1, 2], [0, 1, 2]]
    torch.testing.assert_close(w3, torch.full((2, 3), 1 / 3), rtol=1e-6, atol=0)
    # a tie for the LAST slot only: the lower id wins, the higher is dropped
    lg = torch.tensor([[1.0, 3.0, 2.0, 2.0, 0.0]]).to(torch.bfloat16)
    _, e4 = moe_route_k(lg, 2)
    assert e4.tolist() == [[1, 2]]
    # routing table / active list as the reference's task emits them (routing[e, t] = slot + 1)
    routing, active = moe_routing_tables(torch.tensor([[1, 2], [2, 4]]), 5)
    assert routing.tolist() == [[0, 0], [1, 0], [2, 1], [0, 0], [0, 2]] and active == [1, 2, 4]


def test_moe_mlp_against_dense_float64_and_single_expert_case():
    """moe_mlp_k against a float64 evaluation of the definition out = res + sum_k w_k * W2[e_k] (silu(Wg[e_k] h) * (Wu[e_k] h))
    (tests/runtime_python/test_moe_linear.py:33-61 builds the same per-expert reference), and the special case of one expert
    with weight 1, which is the dense SwiGLU MLP."""
    from oracle.qwen3_ref import linear_k, moe_block_t, moe_mlp_k, moe_route_k, silu_mul_k
    g = torch.Generator().manual_seed(1)
    T, H, E, I, k = 5, 64, 6, 32, 3
    bf = torch.bfloat16
    h = torch.randn(T, H, generator=g).to(bf)
    res = torch.randn(T, H, generator=g).to(bf)
    gu = (0.2 * torch.randn(E, 2 * I, H, generator=g)).to(bf)
    dn = (0.2 * torch.randn(E, H, I, generator=g)).to(bf)
    router = (0.3 * torch.randn(E, H, generator=g)).to(bf)
    w, e = moe_route_k(linear_k(h, router), k)
    out, mid, act, y = moe_mlp_k(h, res, gu, dn, w, e)
    ref = res.double().clone()
    for t in range(T):
        for s in range(k):
            ex = int(e[t, s])
            a = h[t].double() @ gu[ex].double().t()
            m = torch.nn.functional.silu(a[:I]) * a[I:]
            ref[t] += float(w[t, s]) * (m @ dn[ex].double().t())
    torch.testing.assert_close(out.double(), ref, rtol=2e-2, atol=3e-2)
    assert float((out.double() - ref).abs().mean()) < 6e-3  # bf16 rounding of three intermediates, not a structural error
    # slot layout of the intermediates: [T, topk, 2I] with gate rows first (demo_30B_A3B.py:376-420 packs [gate ; up])
    ex = int(e[2, 1])
    torch.testing.assert_close(mid[2, 1].float(), (h[2].float() @ gu[ex].float().t()).to(bf).float())
    assert torch.equal(act[2, 1], silu_mul_k(mid[2, 1, :I], mid[2, 1, I:]))
    # one expert, weight 1: the dense path's unfused operators
    w1, e1 = torch.ones(T, 1), torch.zeros(T, 1, dtype=torch.int64)
    out1 = moe_mlp_k(h, res, gu[:1], dn[:1], w1, e1)[0]
    m1 = linear_k(h, gu[0])
    dense = linear_k(silu_mul_k(m1[:, :I], m1[:, I:]), dn[0])  # bf16(W2 act)
    assert torch.equal(out1, (res.float() + dense.float()).to(bf))
    # the torch-order block (HF algorithm) agrees with the kernel-order one within bf16 tolerance
    blk = res + moe_block_t(h, router, gu, dn, k)
    torch.testing.assert_close(blk.float(), out.float(), rtol=3e-2, atol=6e-2)
