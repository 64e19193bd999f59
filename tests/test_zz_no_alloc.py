"""mk_enqueue_steps_static -- the launch entry point that allocates nothing and keeps all launch scratch in a file-scope
device array -- must give exactly what mk_enqueue_steps gives: same tokens, same logits, bit for bit (the K-split and
split-KV partial sums are combined in a fixed order in both).  Two calls in a row on the same GPU share the array; the
second runs a smaller batch, so whatever the first left behind must not leak into it."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _cfg():
    from oracle.qwen3_ref import Qwen3Config
    # K = 2048 makes the narrow stages of a 16-token iteration split K across workgroups (partial tiles in scratch);
    # contexts beyond 128 positions make the attention stage split KV (partials and arrival counters in scratch)
    return Qwen3Config(hidden_size=2048, num_q_heads=16, num_kv_heads=4, head_dim=128, intermediate_size=2048, num_layers=2, vocab_size=2048)


def _decoder(cfg, w, B, max_seq):
    from demo_qwen3 import Qwen3Decoder, Qwen3Shape
    from oracle.qwen3_ref import rope_tables
    shape = Qwen3Shape(cfg.hidden_size, cfg.num_q_heads, cfg.num_kv_heads, cfg.head_dim, cfg.intermediate_size, cfg.num_layers, cfg.vocab_size, cfg.rope_theta)
    cos, sin = rope_tables(cfg, max_seq)
    wg = {"embed": w["embed"].cuda(), "layers": [{k: v.cuda() for k, v in lw.items()} for lw in w["layers"]],
          "final_norm": w["final_norm"].cuda(), "lm_head": w["lm_head"].cuda()}
    return Qwen3Decoder(shape, wg, max_num_batched_tokens=B, max_num_batched_requests=B, max_seq_length=max_seq, page_size=64, cos_sin=(cos.cuda(), sin.cuda()))


def _run(dec, prompts, static, chunk):
    """Run every request to the end in launches of `chunk` iterations through the chosen entry point; returns the tokens
    and the logits tensor as the last launch left it."""
    from mirage import _capi
    lib = _capi.load()
    dec.load_prompts(prompts)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    fin = ctypes.c_int(0)
    enqueue = lib.mk_enqueue_steps_static if static else lib.mk_enqueue_steps
    launches = 0
    while not fin.value:
        _capi.check(enqueue(dec.mpk._handle, stream, chunk))
        _capi.check(lib.mk_wait(dec.mpk._handle, stream, ctypes.byref(fin)))
        launches += 1
        assert launches < 10000
    assert dec.mpk.stats()["aborted"] == 0
    return dec.meta["tokens"].cpu().clone(), dec.meta["step"].cpu().clone(), dec.logits().cpu().clone()


def test_static_scratch_entry_point_matches_the_allocating_one():
    from oracle.qwen3_ref import make_model_weights, make_prompt
    cfg = _cfg()
    w = make_model_weights(cfg, seed=31)
    max_seq = 200
    big = _decoder(cfg, w, 16, max_seq)     # 16 requests: matrix-core stages with a K split, attention over up to 199 positions
    small = _decoder(cfg, w, 3, max_seq)    # 3 requests: few-token stages, split-KV chunks that span dies
    p_big = [make_prompt(cfg, 20 + 7 * r, 300 + r) for r in range(16)]
    p_small = [make_prompt(cfg, 150 + r, 400 + r) for r in range(3)]
    # the two calls in a row through the static-scratch entry point: first the large batch, then the smaller one
    s_big = _run(big, p_big, static=True, chunk=23)
    s_small = _run(small, p_small, static=True, chunk=5)
    # the same two workloads through the existing entry point
    r_big = _run(big, p_big, static=False, chunk=23)
    r_small = _run(small, p_small, static=False, chunk=5)
    for name, a, b in (("large batch", s_big, r_big), ("small batch after it", s_small, r_small)):
        assert torch.equal(a[1], b[1]) and int(a[1].min()) == max_seq - 1, f"{name}: step counters differ"
        assert torch.equal(a[0], b[0]), f"{name}: tokens differ, first at {(a[0] != b[0]).nonzero()[0].tolist()}"
        assert torch.equal(a[2].view(torch.int16), b[2].view(torch.int16)), f"{name}: logits of the last iteration differ"
    # and once more the large batch, after the small one dirtied the array
    s_big2 = _run(big, p_big, static=True, chunk=200)
    assert torch.equal(s_big2[0], r_big[0]) and torch.equal(s_big2[2].view(torch.int16), r_big[2].view(torch.int16))
    big.mpk.finalize()
    small.mpk.finalize()


def test_static_scratch_entry_point_rejects_what_it_cannot_hold():
    from mirage import _capi
    from oracle.qwen3_ref import Qwen3Config, make_model_weights
    # 64 tokens x 16 kv heads = 1024 (token, kv head) pairs: beyond the 512 the static array holds
    cfg = Qwen3Config(hidden_size=1024, num_q_heads=64, num_kv_heads=16, head_dim=128, intermediate_size=512, num_layers=1, vocab_size=512)
    dec = _decoder(cfg, make_model_weights(cfg, seed=1), 64, 32)
    lib = _capi.load()
    rc = lib.mk_enqueue_steps_static(dec.mpk._handle, ctypes.c_void_p(0), 1)
    assert rc == _capi.MK_EINVAL and b"static launch scratch" in lib.mk_last_error()
    dec.mpk.finalize()
