"""CPU oracle for the Qwen3 decode path -- TEST INFRASTRUCTURE ONLY.

Nothing in the product (fleet-chiplet-megakernel_amd/) may import this module; only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg do, as the checker.

Two restatements of the reference's decode mathematics, written against plain torch CPU ops (plus order="f64", the
same model definition evaluated in float64 without intermediate rounding: the yardstick the two are measured against):

* order="torch"  -- the reference's PyTorch model (demo/qwen3/models/modeling_qwen3.py), which is what
  its greedy loop runs (demo/qwen3/demo.py:1193-1230): every op on bf16 tensors with a bf16 rounding
  after each op, RMSNorm without eps and without fp32 upcast (:49-54), per-head q/k norm (:279-288),
  rotate-half RoPE with bf16 cos/sin (:100-117, rope.py:79-80), KV write at `step` (:300-305),
  scaled_dot_product_attention with GQA (:168-189), SwiGLU (:160-162), bf16 residual adds (:386,394),
  final norm + lm_head (:503,566).
* order="kernel" -- the rounding structure of the reference's MI300 task kernels, which the HIP kernels
  follow: fp32 accumulation and ONE bf16 rounding (round-to-nearest-even) per fused operator:
  RMSNorm bf16((x*r)*w), r = rsqrt(mean(x^2)+1e-6) (tasks/mi300/rmsnorm_mi300.cuh:64-131); linear
  bf16(acc [+ res]) (tasks/mi300/linear_ck_mi300.cuh:582-602); fused SwiGLU bf16(silu(acc_g)*acc_u)
  (tasks/mi300/gang_linear_mi300.cuh:492-498,553-561); q/k norm rounded to bf16 *before* RoPE, RoPE in
  fp32 then bf16 (tasks/mi300/kv_cache_update_mi300.cuh:129-182); softmax in fp32
  (tasks/mi300/paged_attention_decode_minimal_mi300.cuh:236-342); argmax = lowest index of the maximum
  bf16 logit (tasks/mi300/argmax_mi300.cuh:92-157 up to its tie order).

Pinning (tests/test_oracle.py): every function below is checked against closed forms, float64 brute
force on small shapes and invariants (scale invariance, RoPE as a complex rotation, L=1 / constant-K
attention, permutation invariance, planted argmax) -- the reference holds no golden vectors for this
path.  What stays "parity unpinned": the exact summation order inside the reference's ck_tile GEMM
pipelines (third-party, absent from the tree); both restatements accumulate in fp32 like it does.

Mixture of experts (Qwen3-30B-A3B shape): moe_route_k / moe_mlp_k restate the reference's MoE task kernels
(moe_topk_softmax_mi300.cuh, moe_linear_mi300.cuh, moe_mul_sum_add_mi300.cuh) and are pinned against float64
softmax + torch.topk, planted ties, a dense float64 evaluation of the same experts, and the E=1 special case that
reduces to the dense SwiGLU MLP.  moe_block_t restates HF transformers' Qwen3MoeSparseMoeBlock (third-party; the
reference pins 4.57.1, which is not importable here): tests/test_oracle_vs_hf.py checks it against that block of the
installed transformers 5.x on the same bf16 inputs, and checks the dense model composition (order "f64") against
transformers' Qwen3ForCausalLM evaluated in float64; what stays unpinned is only that the pinned 4.57.1 block rounds
at the same points as the 5.x one.
"""
import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

BF16 = torch.bfloat16


@dataclass
class Qwen3Config:
    hidden_size: int = 4096
    num_q_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 12288
    num_layers: int = 36
    vocab_size: int = 151936
    rope_theta: float = 1e6
    rms_eps: float = 1e-6
    max_positions: int = 4096
    # mixture of experts (Qwen3-30B-A3B: 128 experts, top-8, expert width 768); num_experts == 0 -> dense SwiGLU MLP
    num_experts: int = 0
    num_experts_per_tok: int = 0
    moe_intermediate_size: int = 0

    @property
    def q_size(self):
        return self.num_q_heads * self.head_dim

    @property
    def kv_size(self):
        return self.num_kv_heads * self.head_dim


# ----------------------------------------------------------------------------- weights / inputs
def make_layer_weights(cfg: Qwen3Config, gen: torch.Generator, norm_std: float = 0.0):
    """Linear weights ~ N(0, 0.02) in bf16; norm weights = 1 (+ N(0, norm_std) when norm_std > 0)."""
    H, I, D = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim

    def lin(n, k):
        return (torch.randn(n, k, generator=gen, dtype=torch.float32) * 0.02).to(BF16)

    def norm(n):
        w = torch.ones(n, dtype=torch.float32)
        if norm_std > 0:
            w = w + torch.randn(n, generator=gen, dtype=torch.float32) * norm_std
        return w.to(BF16)

    w = {
        "input_norm": norm(H), "q_proj": lin(cfg.q_size, H), "k_proj": lin(cfg.kv_size, H), "v_proj": lin(cfg.kv_size, H),
        "q_norm": norm(D), "k_norm": norm(D), "o_proj": lin(H, cfg.q_size), "post_norm": norm(H),
    }
    if cfg.num_experts > 0:
        E, MI = cfg.num_experts, cfg.moe_intermediate_size
        # expert tensors as the reference driver packs them (demo/qwen3/demo_30B_A3B.py:376-420):
        # gate_up_proj [E, 2*MI, H] = [gate ; up] per expert, down_proj [E, H, MI]
        w["router"] = lin(E, H)
        w["gate_up_proj"] = (torch.randn(E, 2 * MI, H, generator=gen, dtype=torch.float32) * 0.02).to(BF16)
        w["down_proj"] = (torch.randn(E, H, MI, generator=gen, dtype=torch.float32) * 0.02).to(BF16)
    else:
        w.update({"gate_proj": lin(I, H), "up_proj": lin(I, H), "down_proj": lin(H, I)})
    return w


def make_model_weights(cfg: Qwen3Config, seed: int = 0, norm_std: float = 0.0):
    gen = torch.Generator().manual_seed(seed)
    w = {"embed": (torch.randn(cfg.vocab_size, cfg.hidden_size, generator=gen, dtype=torch.float32) * 0.02).to(BF16)}
    w["layers"] = [make_layer_weights(cfg, gen, norm_std) for _ in range(cfg.num_layers)]
    w["final_norm"] = torch.ones(cfg.hidden_size, dtype=torch.float32).to(BF16)
    w["lm_head"] = (torch.randn(cfg.vocab_size, cfg.hidden_size, generator=gen, dtype=torch.float32) * 0.02).to(BF16)
    return w


def make_prompt(cfg: Qwen3Config, length: int, seed: int):
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg.vocab_size, (length,), generator=gen, dtype=torch.int64)


def rope_tables(cfg: Qwen3Config, n_pos: int = None):
    """bf16 cos/sin tables [n_pos, head_dim] with both halves equal (modeling_qwen3.py:100-117; inv_freq =
    theta^(-2i/D), the HF "default" rope init)."""
    n_pos = n_pos or cfg.max_positions
    D = cfg.head_dim
    inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    freqs = torch.arange(n_pos, dtype=torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(BF16), emb.sin().to(BF16)


# ----------------------------------------------------------------------------- kernel-order operators
def rmsnorm_k(x, w, eps=1e-6):
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return ((xf * r) * w.float()).to(BF16)


def linear_k(x, W, res=None, acc=torch.float32):
    """bf16(x W^T [+ res]) accumulated in `acc` (fp32: what the kernels do; float64: the same rounding points with exact
    sums, used to measure how far two legitimate summation orders drift apart through a deep model)."""
    y = x.to(acc) @ W.to(acc).t()
    if res is not None:
        y = y + res.to(acc)
    return y.to(BF16)


def silu_mul_f32(g, u):
    return g / (1.0 + torch.exp(-g)) * u


def linear_silu_k(x, Wg, Wu, acc=torch.float32):
    xf = x.to(acc)
    return silu_mul_f32(xf @ Wg.to(acc).t(), xf @ Wu.to(acc).t()).to(BF16)


def silu_mul_k(gate_bf16, up_bf16):
    return silu_mul_f32(gate_bf16.float(), up_bf16.float()).to(BF16)


def moe_route_margin(logits_bf16, topk: int):
    """Relative gap (p_k - p_{k+1}) / p_k between the last selected and the first rejected router probability, per token.
    Top-k routing is discontinuous: where this gap is within a bf16 rounding of the logits, a 1-ulp difference upstream
    legitimately selects another expert, so parity tests compare outputs only where the gap is comfortable."""
    p = torch.softmax(logits_bf16.float(), -1).sort(-1, descending=True).values
    if p.shape[-1] <= topk:
        return torch.ones(p.shape[0])
    return (p[:, topk - 1] - p[:, topk]) / p[:, topk - 1]


def moe_route_k(logits_bf16, topk: int):
    """Router of the reference's MoE path (tasks/mi300/moe_topk_softmax_mi300.cuh:124-213): fp32 softmax over ALL
    experts, `topk` rounds of arg-max where equal probabilities go to the lower expert id, weights renormalised by
    the sum of the selected probabilities.  Returns (weights fp32 [T, topk], experts int64 [T, topk]) in slot order."""
    x = logits_bf16.float()
    p = torch.exp(x - x.max(-1, keepdim=True).values)
    p = p * (1.0 / p.sum(-1, keepdim=True))
    T, E = p.shape
    w = torch.zeros(T, topk, dtype=torch.float32)
    e = torch.zeros(T, topk, dtype=torch.int64)
    q = p.clone()
    for s in range(topk):
        best = q.max(-1).values
        idx = (q == best[:, None]).float().argmax(-1)  # first (lowest) index attaining the maximum
        w[:, s], e[:, s] = best, idx
        q[torch.arange(T), idx] = -10000.0
    return w * (1.0 / w.sum(-1, keepdim=True)), e


def moe_routing_tables(experts, num_experts: int):
    """The routing table / mask tensors the reference's router task emits (moe_topk_softmax_mi300.cuh:176-229):
    routing[e, t] = 1 + slot if expert e serves token t else 0; mask = ids of the active experts (any order) with
    their count at index num_experts."""
    T, topk = experts.shape
    routing = torch.zeros(num_experts, T, dtype=torch.int32)
    for t in range(T):
        for s in range(topk):
            routing[experts[t, s], t] = s + 1
    active = sorted(set(experts.flatten().tolist()))
    return routing, active


def moe_mlp_k(h, x_res, gate_up, down, weights, experts, acc=torch.float32):
    """Kernel-order expert MLP + combine on T tokens.  h: normalised input [T, H] bf16; x_res: residual [T, H] bf16;
    gate_up [E, 2I, H], down [E, H, I].  Rounding points follow the reference's task sequence
    (demo/qwen3/demo_30B_A3B.py:697-754): W13 output [T, topk, 2I] rounded to bf16
    (tasks/mi300/moe_linear_mi300.cuh:53-295), SwiGLU on those bf16 values -> bf16, W2 output [T, topk, H] rounded to
    bf16, then out = bf16(res + sum_k w_k * y_k) accumulated in fp32 in slot order
    (tasks/mi300/moe_mul_sum_add_mi300.cuh:41-54).  `acc`: accumulation type of the two expert linears (see linear_k).
    Returns (out, mid, act, y)."""
    T, topk = experts.shape
    I2 = gate_up.shape[1]
    H = down.shape[1]
    mid = torch.zeros(T, topk, I2, dtype=BF16)
    act = torch.zeros(T, topk, I2 // 2, dtype=BF16)
    y = torch.zeros(T, topk, H, dtype=BF16)
    out = torch.zeros(T, H, dtype=BF16)
    for t in range(T):
        acc = x_res[t].float()
        for s in range(topk):
            e = int(experts[t, s])
            mid[t, s] = (h[t].to(acc) @ gate_up[e].to(acc).t()).to(BF16)
            act[t, s] = silu_mul_k(mid[t, s, :I2 // 2], mid[t, s, I2 // 2:])
            y[t, s] = (act[t, s].to(acc) @ down[e].to(acc).t()).to(BF16)
            acc = acc + y[t, s].float() * weights[t, s]
        out[t] = acc.to(BF16)
    return out, mid, act, y


def moe_block_t(h, router, gate_up, down, topk: int):
    """torch-order sparse MoE block = HF transformers 4.57.1 Qwen3MoeSparseMoeBlock.forward with norm_topk_prob=True
    (third-party; restated from its published algorithm, PARITY UNPINNED): bf16 router linear, fp32 softmax, top-k,
    renormalise, routing weights cast to bf16, per-expert SwiGLU MLP in bf16 scaled by the bf16 weight and
    index-added into a bf16 buffer in ascending expert order."""
    T, H = h.shape
    logits = F.linear(h, router)
    rw = F.softmax(logits, dim=1, dtype=torch.float)
    rw, sel = torch.topk(rw, topk, dim=-1)
    rw = (rw / rw.sum(dim=-1, keepdim=True)).to(h.dtype)
    out = torch.zeros(T, H, dtype=h.dtype)
    I = gate_up.shape[1] // 2
    for e in sorted(set(sel.flatten().tolist())):
        tok, slot = torch.where(sel == e)
        cur = h[tok]
        y = F.linear(F.silu(F.linear(cur, gate_up[e, :I])) * F.linear(cur, gate_up[e, I:]), down[e])
        out.index_add_(0, tok, (y * rw[tok, slot, None]).to(h.dtype))
    return out


def head_norm_rope_k(x, w, cos_row, sin_row, eps=1e-6, qk_norm=True, rope=True):
    """x: [..., D] bf16 head rows; cos_row/sin_row: [..., D] bf16 for each row's position."""
    D = x.shape[-1]
    xf = x.float()
    if qk_norm:
        r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
        xf = ((xf * r) * w.float()).to(BF16).float()
    if rope:
        h = D // 2
        x0, x1 = xf[..., :h], xf[..., h:]
        c, s = cos_row.float()[..., :h], sin_row.float()[..., :h]
        xf = torch.cat((x0 * c - x1 * s, x0 * s + x1 * c), dim=-1)
    return xf.to(BF16)


def attention_k(q, K, V):
    """q: [nq, D] bf16; K, V: [L, nkv, D] bf16 -> [nq, D] bf16.  fp32 softmax(q K^T / sqrt(D)) V."""
    nq, D = q.shape
    L, nkv, _ = K.shape
    g = nq // nkv
    qf = q.float().view(nkv, g, D)
    Kf = K.float().permute(1, 0, 2)  # [nkv, L, D]
    Vf = V.float().permute(1, 0, 2)
    s = torch.einsum("hgd,hld->hgl", qf, Kf) / math.sqrt(D)
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hgl,hld->hgd", p, Vf)
    return o.reshape(nq, D).to(BF16)


def argmax_k(logits_bf16):
    """Lowest index attaining the maximum, per row."""
    lf = logits_bf16.float()
    mx = lf.max(dim=-1, keepdim=True).values
    idx = torch.arange(lf.shape[-1]).expand_as(lf)
    return torch.where(lf == mx, idx, torch.full_like(idx, lf.shape[-1])).min(dim=-1).values


# ----------------------------------------------------------------------------- torch-order operators
def rmsnorm_t(x, w):
    var = x.pow(2).mean(-1, keepdim=True)
    return w * (x * torch.rsqrt(var))


def rope_t(x, cos_row, sin_row):
    h = x.shape[-1] // 2
    x1, x2 = x[..., :h], x[..., h:]
    c, s = cos_row[..., :h], sin_row[..., :h]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


# ----------------------------------------------------------------------------- model
class KVCache:
    """Contiguous per-request cache [layers, max_seq, nkv, D] (the reference's torch path uses one page)."""

    def __init__(self, cfg: Qwen3Config, max_seq: int, dtype=BF16):
        self.k = torch.zeros(cfg.num_layers, max_seq, cfg.num_kv_heads, cfg.head_dim, dtype=dtype)
        self.v = torch.zeros_like(self.k)


class Qwen3Oracle:
    def __init__(self, cfg: Qwen3Config, weights: dict, order: str = "kernel", rope=None, acc=torch.float32):
        """rope: optional (cos, sin) tables [positions, head_dim] replacing the bf16 ones (the float64 order can be given
        unrounded tables to be compared with an independent float64 evaluation).  acc: accumulation type of the
        kernel-order linears (see linear_k)."""
        assert order in ("kernel", "torch", "f64")
        self.cfg, self.w, self.order, self.acc = cfg, weights, order, acc
        self.cos, self.sin = rope if rope is not None else rope_tables(cfg)
        self.route_margins = []  # mixture of experts: smallest routing gap of every layer call since the last forward()

    # one decoder layer on T new tokens of ONE request at absolute positions pos0..pos0+T-1
    def layer(self, li: int, x, cache: KVCache, pos0: int):
        cfg, W = self.cfg, self.w["layers"][li]
        T = x.shape[0]
        D, nq, nkv = cfg.head_dim, cfg.num_q_heads, cfg.num_kv_heads
        pos = torch.arange(pos0, pos0 + T)
        cos, sin = self.cos[pos][:, None, :], self.sin[pos][:, None, :]
        if self.order == "kernel":
            acc = self.acc
            h = rmsnorm_k(x, W["input_norm"], cfg.rms_eps)
            q, k, v = linear_k(h, W["q_proj"], acc=acc), linear_k(h, W["k_proj"], acc=acc), linear_k(h, W["v_proj"], acc=acc)
            q = head_norm_rope_k(q.view(T, nq, D), W["q_norm"], cos, sin, cfg.rms_eps)
            k = head_norm_rope_k(k.view(T, nkv, D), W["k_norm"], cos, sin, cfg.rms_eps)
            cache.k[li, pos0:pos0 + T] = k
            cache.v[li, pos0:pos0 + T] = v.view(T, nkv, D)
            a = torch.stack([attention_k(q[t], cache.k[li, :pos0 + t + 1], cache.v[li, :pos0 + t + 1]) for t in range(T)])
            x = linear_k(a.view(T, nq * D), W["o_proj"], res=x, acc=acc)
            h = rmsnorm_k(x, W["post_norm"], cfg.rms_eps)
            if cfg.num_experts > 0:
                gate = linear_k(h, W["router"], acc=acc)
                self.route_margins.append(float(moe_route_margin(gate, cfg.num_experts_per_tok).min()))
                wts, exp = moe_route_k(gate, cfg.num_experts_per_tok)
                return moe_mlp_k(h, x, W["gate_up_proj"], W["down_proj"], wts, exp, acc=acc)[0]
            m = linear_silu_k(h, W["gate_proj"], W["up_proj"], acc=acc)
            return linear_k(m, W["down_proj"], res=x, acc=acc)
        if self.order == "f64":
            return self._layer_f64(li, x, cache, pos0)
        # torch order
        h = rmsnorm_t(x, W["input_norm"])
        q, k, v = F.linear(h, W["q_proj"]), F.linear(h, W["k_proj"]), F.linear(h, W["v_proj"])
        q = rope_t(rmsnorm_t(q.view(T, nq, D), W["q_norm"]), cos, sin)
        k = rope_t(rmsnorm_t(k.view(T, nkv, D), W["k_norm"]), cos, sin)
        cache.k[li, pos0:pos0 + T] = k
        cache.v[li, pos0:pos0 + T] = v.view(T, nkv, D)
        L = pos0 + T
        qs = q.permute(1, 0, 2)
        ks = cache.k[li, :L].permute(1, 0, 2)
        vs = cache.v[li, :L].permute(1, 0, 2)
        if T > 1:
            assert pos0 == 0, "the reference only prefills from position 0"
            a = F.scaled_dot_product_attention(qs, ks, vs, is_causal=True, enable_gqa=True)
        else:
            a = F.scaled_dot_product_attention(qs, ks, vs, is_causal=False, enable_gqa=True)
        a = a.permute(1, 0, 2).reshape(T, nq * D)
        x = x + F.linear(a, W["o_proj"])
        h = rmsnorm_t(x, W["post_norm"])
        if cfg.num_experts > 0:
            return x + moe_block_t(h, W["router"], W["gate_up_proj"], W["down_proj"], cfg.num_experts_per_tok)
        m = F.silu(F.linear(h, W["gate_proj"])) * F.linear(h, W["up_proj"])
        return x + F.linear(m, W["down_proj"])

    def _layer_f64(self, li: int, x, cache, pos0: int):
        """The dense layer's definition evaluated in float64 with no intermediate rounding (the same bf16 weights and
        cos/sin tables, eps as the kernels): the yardstick both rounding orders are measured against.  `cache` must be a
        KVCache created with dtype=torch.float64."""
        cfg, W = self.cfg, {k: v.double() for k, v in self.w["layers"][li].items()}
        assert cfg.num_experts == 0
        T, D, nq, nkv = x.shape[0], cfg.head_dim, cfg.num_q_heads, cfg.num_kv_heads
        pos = torch.arange(pos0, pos0 + T)
        cos, sin = self.cos[pos][:, None, :].double(), self.sin[pos][:, None, :].double()
        norm = lambda v, w: v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + cfg.rms_eps) * w
        h = norm(x, W["input_norm"])
        q, k, v = h @ W["q_proj"].t(), h @ W["k_proj"].t(), h @ W["v_proj"].t()
        q = rope_t(norm(q.view(T, nq, D), W["q_norm"]), cos, sin)
        k = rope_t(norm(k.view(T, nkv, D), W["k_norm"]), cos, sin)
        cache.k[li, pos0:pos0 + T] = k
        cache.v[li, pos0:pos0 + T] = v.view(T, nkv, D)
        outs = []
        for t in range(T):
            L = pos0 + t + 1
            Kf = cache.k[li, :L].permute(1, 0, 2).repeat_interleave(nq // nkv, 0)  # [nq, L, D]
            Vf = cache.v[li, :L].permute(1, 0, 2).repeat_interleave(nq // nkv, 0)
            p = torch.softmax(torch.einsum("hd,hld->hl", q[t], Kf) / math.sqrt(D), -1)
            outs.append(torch.einsum("hl,hld->hd", p, Vf).reshape(nq * D))
        x = x + torch.stack(outs) @ W["o_proj"].t()
        h = norm(x, W["post_norm"])
        g, u = h @ W["gate_proj"].t(), h @ W["up_proj"].t()
        return x + (g / (1.0 + torch.exp(-g)) * u) @ W["down_proj"].t()

    def forward(self, ids, cache: KVCache, pos0: int):
        """ids: [T] int64 tokens of one request at positions pos0.. -> logits [T, vocab] bf16 (float64 for order "f64")."""
        x = self.w["embed"][ids]
        self.route_margins = []
        if self.order == "f64":
            x = x.double()
            for li in range(self.cfg.num_layers):
                x = self._layer_f64(li, x, cache, pos0)
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.cfg.rms_eps) * self.w["final_norm"].double()
            return x @ self.w["lm_head"].double().t()
        for li in range(self.cfg.num_layers):
            x = self.layer(li, x, cache, pos0)
        if self.order == "kernel":
            h = rmsnorm_k(x, self.w["final_norm"], self.cfg.rms_eps)
            self.last_hidden = h  # the normalised final hidden state of the last forward()
            return linear_k(h, self.w["lm_head"], acc=self.acc)
        return F.linear(rmsnorm_t(x, self.w["final_norm"]), self.w["lm_head"])
