"""CPU oracle for the Qwen3 decode path -- TEST INFRASTRUCTURE ONLY.

Nothing in the product (fleet-chiplet-megakernel_amd/) may import this module; only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg do, as the checker.

Two restatements of the reference's decode mathematics, written against plain torch CPU ops:

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

    return {
        "input_norm": norm(H), "q_proj": lin(cfg.q_size, H), "k_proj": lin(cfg.kv_size, H), "v_proj": lin(cfg.kv_size, H),
        "q_norm": norm(D), "k_norm": norm(D), "o_proj": lin(H, cfg.q_size),
        "post_norm": norm(H), "gate_proj": lin(I, H), "up_proj": lin(I, H), "down_proj": lin(H, I),
    }


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


def linear_k(x, W, res=None):
    y = x.float() @ W.float().t()
    if res is not None:
        y = y + res.float()
    return y.to(BF16)


def silu_mul_f32(g, u):
    return g / (1.0 + torch.exp(-g)) * u


def linear_silu_k(x, Wg, Wu):
    xf = x.float()
    return silu_mul_f32(xf @ Wg.float().t(), xf @ Wu.float().t()).to(BF16)


def silu_mul_k(gate_bf16, up_bf16):
    return silu_mul_f32(gate_bf16.float(), up_bf16.float()).to(BF16)


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

    def __init__(self, cfg: Qwen3Config, max_seq: int):
        self.k = torch.zeros(cfg.num_layers, max_seq, cfg.num_kv_heads, cfg.head_dim, dtype=BF16)
        self.v = torch.zeros_like(self.k)


class Qwen3Oracle:
    def __init__(self, cfg: Qwen3Config, weights: dict, order: str = "kernel"):
        assert order in ("kernel", "torch")
        self.cfg, self.w, self.order = cfg, weights, order
        self.cos, self.sin = rope_tables(cfg)

    # one decoder layer on T new tokens of ONE request at absolute positions pos0..pos0+T-1
    def layer(self, li: int, x, cache: KVCache, pos0: int):
        cfg, W = self.cfg, self.w["layers"][li]
        T = x.shape[0]
        D, nq, nkv = cfg.head_dim, cfg.num_q_heads, cfg.num_kv_heads
        pos = torch.arange(pos0, pos0 + T)
        cos, sin = self.cos[pos][:, None, :], self.sin[pos][:, None, :]
        if self.order == "kernel":
            h = rmsnorm_k(x, W["input_norm"], cfg.rms_eps)
            q, k, v = linear_k(h, W["q_proj"]), linear_k(h, W["k_proj"]), linear_k(h, W["v_proj"])
            q = head_norm_rope_k(q.view(T, nq, D), W["q_norm"], cos, sin, cfg.rms_eps)
            k = head_norm_rope_k(k.view(T, nkv, D), W["k_norm"], cos, sin, cfg.rms_eps)
            cache.k[li, pos0:pos0 + T] = k
            cache.v[li, pos0:pos0 + T] = v.view(T, nkv, D)
            a = torch.stack([attention_k(q[t], cache.k[li, :pos0 + t + 1], cache.v[li, :pos0 + t + 1]) for t in range(T)])
            x = linear_k(a.view(T, nq * D), W["o_proj"], res=x)
            h = rmsnorm_k(x, W["post_norm"], cfg.rms_eps)
            m = linear_silu_k(h, W["gate_proj"], W["up_proj"])
            return linear_k(m, W["down_proj"], res=x)
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
        m = F.silu(F.linear(h, W["gate_proj"])) * F.linear(h, W["up_proj"])
        return x + F.linear(m, W["down_proj"])

    def forward(self, ids, cache: KVCache, pos0: int):
        """ids: [T] int64 tokens of one request at positions pos0.. -> logits [T, vocab] bf16."""
        x = self.w["embed"][ids]
        for li in range(self.cfg.num_layers):
            x = self.layer(li, x, cache, pos0)
        if self.order == "kernel":
            h = rmsnorm_k(x, self.w["final_norm"], self.cfg.rms_eps)
            return linear_k(h, self.w["lm_head"])
        return F.linear(rmsnorm_t(x, self.w["final_norm"]), self.w["lm_head"])

    def greedy(self, prompt, n_new: int, max_seq: int, teacher=None, token_by_token_prefill=False):
        """Prefill then greedy decode (demo.py:1193-1212).  Returns (tokens [len+n_new], logits per decode step).
        teacher: optional ids to force-feed instead of the argmax (teacher forcing)."""
        cache = KVCache(self.cfg, max_seq)
        P = prompt.shape[0]
        toks = prompt.tolist()
        logits_out = []
        if token_by_token_prefill:
            for p in range(P):
                lg = self.forward(prompt[p:p + 1], cache, p)
        else:
            lg = self.forward(prompt, cache, 0)[-1:]
        for i in range(n_new):
            logits_out.append(lg[0])
            nxt = int(argmax_k(lg)[0]) if self.order == "kernel" else int(lg[0].argmax(-1))
            toks.append(nxt)
            feed = nxt if teacher is None else int(teacher[i])
            if i + 1 < n_new:
                lg = self.forward(torch.tensor([feed]), cache, P + i)
        return torch.tensor(toks), logits_out
