"""Headline configuration 2 (one Qwen3-8B-shaped decoder layer, 512 cached positions, one new token, BS=1) and smaller /
multi-token variants of the same layer, GPU vs the kernel-order CPU oracle, through the PersistentKernel API."""
import pytest
import torch

from helpers import check_layer_stages as _check

pytestmark = pytest.mark.gpu


def _run_layer(cfg, L_cached, n_new, mode, seed=0, norm_std=0.02, mutate=None, batch_tokens=None, single_weight_copy=None):
    """One request with L_cached positions already in the KV cache and n_new new tokens in this pass."""
    from demo_qwen3 import Qwen3Decoder, Qwen3Shape
    from oracle.qwen3_ref import KVCache, Qwen3Oracle, make_layer_weights, rope_tables
    g = torch.Generator().manual_seed(seed)
    lw = make_layer_weights(cfg, g, norm_std=norm_std)
    if mutate is not None:
        mutate(lw)
    hidden = torch.randn(n_new, cfg.hidden_size, generator=g).to(torch.bfloat16)
    max_seq = L_cached + n_new + 8
    cache = KVCache(cfg, max_seq)
    cache.k[0, :L_cached] = torch.randn(L_cached, cfg.num_kv_heads, cfg.head_dim, generator=g).to(torch.bfloat16)
    cache.v[0, :L_cached] = torch.randn(L_cached, cfg.num_kv_heads, cfg.head_dim, generator=g).to(torch.bfloat16)
    shape = Qwen3Shape(cfg.hidden_size, cfg.num_q_heads, cfg.num_kv_heads, cfg.head_dim, cfg.intermediate_size, 1, 1024, cfg.rope_theta)
    dev = "cuda"
    w = {"embed": torch.zeros(1024, cfg.hidden_size, dtype=torch.bfloat16, device=dev),
         "layers": [{k: v.to(dev) for k, v in lw.items()}],
         "final_norm": torch.ones(cfg.hidden_size, dtype=torch.bfloat16, device=dev),
         "lm_head": torch.zeros(1024, cfg.hidden_size, dtype=torch.bfloat16, device=dev)}
    cos, sin = rope_tables(cfg, max(max_seq, 16))
    page_size = 64
    n_pages = (max_seq + page_size - 1) // page_size
    dec = Qwen3Decoder(shape, w, max_num_batched_tokens=batch_tokens or max(n_new, 1), max_num_batched_requests=1, max_seq_length=max_seq, single_weight_copy=single_weight_copy,
                       page_size=page_size, max_num_pages=n_pages + 3, mode=mode, cos_sin=(cos.to(dev), sin.to(dev)), with_head=False,
                       max_tokens_per_request=max(8, n_new))
    if single_weight_copy:
        released = dec.mpk.release_row_major_weights()
        assert len(released) == 7  # q, k, v, o, gate, up, down (the zero LM head of this one-layer graph is not lowered)
        for k in ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"):
            w["layers"][0][k].fill_(float("nan"))  # whoever still reads the row-major tensors will show it
    # scatter the cached positions over non-trivially ordered pages: request slot 0 owns pages [n_pages+2, n_pages+1, ... ]
    pages = list(range(n_pages + 2, 2, -1))[:n_pages]
    dec.meta["paged_kv_indptr_buffer"].copy_(torch.tensor([0, n_pages], dtype=torch.int32))
    idx = torch.zeros(dec.max_pages, dtype=torch.int32)
    idx[:n_pages] = torch.tensor(pages, dtype=torch.int32)
    dec.meta["paged_kv_indices_buffer"].copy_(idx)
    kc, vc = torch.zeros_like(dec.k_cache[0].cpu()), torch.zeros_like(dec.v_cache[0].cpu())
    for p in range(L_cached):
        kc[pages[p // page_size], p % page_size] = cache.k[0, p]
        vc[pages[p // page_size], p % page_size] = cache.v[0, p]
    dec.k_cache[0].copy_(kc)
    dec.v_cache[0].copy_(vc)
    # run only the layer's stages: feed hidden through the embedding table trick (ids pick rows of a table = hidden)
    dec.w["embed"][:n_new].copy_(hidden.to(dev))
    dec.meta["input_tokens"][:n_new].copy_(torch.arange(n_new, dtype=torch.int64).view(-1, 1))
    torch.cuda.synchronize()
    dec.mpk.run_once([0] * n_new, list(range(L_cached, L_cached + n_new)))
    out_gpu = dec.t["hidden_out"].to_torch()[:n_new].cpu()
    attn_gpu = dec.t["attn_out"].to_torch()[:n_new].cpu()
    qkv_gpu = dec.t["attn_in"].to_torch()[:n_new].cpu()
    qws_gpu = dec.t["q_ws"].to_torch()[:n_new].cpu()
    extra = {k: dec.t[k].to_torch()[:n_new].cpu() for k in ('attn_proj_out', 'silu_mul_out', 'rmsnorm_out')}
    k_after = dec.k_cache[0].cpu()
    v_after = dec.v_cache[0].cpu()
    # oracle
    ocfg = cfg
    orc = Qwen3Oracle(ocfg, {"layers": [lw]}, "kernel")
    orc.cos, orc.sin = cos, sin
    import copy
    cache_ref = copy.deepcopy(cache)
    out_ref = orc.layer(0, hidden, cache_ref, L_cached)
    res = dict(out_gpu=out_gpu, out_ref=out_ref, attn_gpu=attn_gpu, qkv_gpu=qkv_gpu, qws_gpu=qws_gpu, cache=cache, lw=lw, hidden=hidden, cos=cos, sin=sin, k_after=k_after, v_after=v_after,
               pages=pages, page_size=page_size, extra=extra, stats=dec.mpk.stats(), program=dec.mpk.describe_program())
    dec.mpk.finalize()
    return res


@pytest.mark.parametrize("mode", ["fleet", "mpk"])
def test_config2_full_width_layer(mode):
    from oracle.qwen3_ref import Qwen3Config
    cfg = Qwen3Config(num_layers=1)
    res = _run_layer(cfg, 512, 1, mode)
    _check(res, cfg, 512, 1)


@pytest.mark.parametrize("L_cached,n_new", [(0, 1), (1, 1), (31, 1), (33, 1), (200, 1), (1100, 1)])
def test_small_layer_decode_lengths(L_cached, n_new):
    from oracle.qwen3_ref import Qwen3Config
    cfg = Qwen3Config(hidden_size=1024, num_q_heads=8, num_kv_heads=2, head_dim=128, intermediate_size=1536, num_layers=1)
    res = _run_layer(cfg, L_cached, n_new, "fleet", seed=L_cached + 1)
    _check(res, cfg, L_cached, n_new)


def test_v_append_exact_and_qkv_matches():
    from oracle.qwen3_ref import Qwen3Config
    cfg = Qwen3Config(hidden_size=1024, num_q_heads=8, num_kv_heads=2, head_dim=128, intermediate_size=1536, num_layers=1)
    res = _run_layer(cfg, 70, 1, "fleet", seed=5)
    pages, ps = res["pages"], res["page_size"]
    # V row in the cache must be the exact bf16 v slice of the QKV output (per kv-head group layout [q x4 ; k ; v])
    qkv = res["qkv_gpu"][0].view(cfg.num_kv_heads, (cfg.num_q_heads // cfg.num_kv_heads) + 2, cfg.head_dim)
    v_new = qkv[:, -1, :]
    assert torch.equal(res["v_after"][pages[70 // ps], 70 % ps], v_new)


@pytest.mark.parametrize("L_cached,n_new", [(0, 5), (0, 8), (70, 8), (300, 3), (63, 2)])
def test_small_layer_prefill_chunks(L_cached, n_new):
    """Several new tokens of one request in one pass (chunked prefill): causal attention inside the chunk, MFMA linears."""
    from oracle.qwen3_ref import Qwen3Config
    cfg = Qwen3Config(hidden_size=1024, num_q_heads=8, num_kv_heads=2, head_dim=128, intermediate_size=1536, num_layers=1)
    res = _run_layer(cfg, L_cached, n_new, "fleet", seed=100 + L_cached + n_new)
    _check(res, cfg, L_cached, n_new)


def test_full_width_layer_prefill_chunk_mpk_mode():
    from oracle.qwen3_ref import Qwen3Config
    cfg = Qwen3Config(num_layers=1)
    res = _run_layer(cfg, 40, 8, "mpk", seed=9)
    _check(res, cfg, 40, 8)


@pytest.mark.parametrize("n_new", [2, 4, 7])
def test_full_width_layer_few_tokens_fleet_mode(n_new):
    """Full-width layer with 2..8 new tokens in the gang configuration: the few-token linears (token rows in LDS, fused
    RMSNorm, fused SwiGLU, residual travelling with the rows) for every token-count instantiation."""
    from oracle.qwen3_ref import Qwen3Config
    cfg = Qwen3Config(num_layers=1)
    res = _run_layer(cfg, 24, n_new, "fleet", seed=40 + n_new)
    _check(res, cfg, 24, n_new)
