"""The host-driven modes of the persistent kernel (reference: MODE_ONLINE / MODE_ONLINE_NOTOKEN / MODE_ONEPASS,
include/mirage/persistent_kernel/persistent_kernel.cuh:538-582) against the offline mode on the same small model:

* online_notoken -- one pass per launch over the batch the HOST described in the meta tensors (the serving-loop mode of
  mirage/mpk/mpk.py): a host loop that does the scheduler's job must reproduce the offline run's tokens exactly;
* online -- one request whose tokens the host wrote: the kernel walks them num_new_tokens[0] at a time (teacher
  forcing); feeding it the offline run's tokens must reproduce the offline run's choice at every position."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _cfg():
    from oracle.qwen3_ref import Qwen3Config
    return Qwen3Config(hidden_size=1024, num_q_heads=8, num_kv_heads=2, head_dim=128, intermediate_size=1536, num_layers=2, vocab_size=2048)


def _decoder(cfg, w, **kw):
    from demo_qwen3 import Qwen3Decoder, Qwen3Shape
    from oracle.qwen3_ref import rope_tables
    shape = Qwen3Shape(cfg.hidden_size, cfg.num_q_heads, cfg.num_kv_heads, cfg.head_dim, cfg.intermediate_size, cfg.num_layers, cfg.vocab_size, cfg.rope_theta)
    cos, sin = rope_tables(cfg, max(kw.get("max_seq_length", 64), 16))
    wg = {"embed": w["embed"].cuda(), "layers": [{k: v.cuda() for k, v in lw.items()} for lw in w["layers"]],
          "final_norm": w["final_norm"].cuda(), "lm_head": w["lm_head"].cuda()}
    return Qwen3Decoder(shape, wg, cos_sin=(cos.cuda(), sin.cuda()), **kw)


def test_online_notoken_host_loop_reproduces_offline_tokens():
    """The host plays scheduler with the C restatement of the reference's offline scheduler: every iteration it writes the
    batch that scheduler forms into the meta tensors and launches one pass.  Same batches, same page assignment, same
    kernel forms as the on-GPU scheduler's run -- so the tokens must be identical, position by position."""
    import numpy as np
    from oracle.qwen3_ref import make_model_weights, make_prompt
    from oracle.sched_ref import SchedulerOracle
    cfg = _cfg()
    w = make_model_weights(cfg, seed=41)
    R, B, total, max_seq, PS = 3, 8, 5, 40, 16
    prompts = [make_prompt(cfg, n, 500 + i) for i, n in enumerate((5, 11, 8, 3, 17))]
    pages = R * ((max_seq + PS - 1) // PS)
    off = _decoder(cfg, w, max_num_batched_tokens=B, max_num_batched_requests=R, max_seq_length=max_seq, page_size=PS, total_requests=total)
    ref_tokens, ref_steps = off.generate(prompts)
    off.mpk.finalize()
    on = _decoder(cfg, w, max_num_batched_tokens=B, max_num_batched_requests=R, max_seq_length=max_seq, page_size=PS, total_requests=total,
                  kernel_mode="online_notoken")
    orc = SchedulerOracle([p.tolist() for p in prompts], R, B, pages, PS, max_seq)
    m = on.meta
    out_prev, iters = None, 0
    while True:
        n = orc.step(out_prev)
        if n == 0:
            break
        m["input_tokens"].copy_(torch.from_numpy(orc["input_tokens"]).view(-1, 1))
        m["qo_indptr_buffer"].copy_(torch.from_numpy(orc["qo_indptr"]))
        m["paged_kv_indptr_buffer"].copy_(torch.from_numpy(orc["kv_indptr"]))
        m["paged_kv_indices_buffer"].copy_(torch.from_numpy(orc["kv_indices"]))
        m["paged_kv_last_page_len_buffer"].copy_(torch.from_numpy(orc["kv_last_page_len"]))
        torch.cuda.synchronize()
        on.mpk()  # one pass over the batch just described
        out_prev = m["output_tokens"].cpu().numpy().reshape(-1)
        iters += 1
        assert iters < 1000
    assert np.array_equal(orc["tokens"], ref_tokens.numpy()), "host-driven passes and the on-GPU scheduler's run disagree"
    assert np.array_equal(orc["step"], ref_steps.numpy())
    assert on.mpk.stats()["aborted"] == 0
    on.mpk.finalize()


def test_online_mode_walks_host_written_tokens():
    from oracle.qwen3_ref import make_model_weights, make_prompt
    cfg = _cfg()
    w = make_model_weights(cfg, seed=42)
    max_seq, P = 36, 9
    prompt = make_prompt(cfg, P, 7)
    off = _decoder(cfg, w, max_num_batched_tokens=1, max_seq_length=max_seq, page_size=16)
    ref_tokens, _ = off.generate([prompt])
    off.mpk.finalize()
    ref = ref_tokens[0]
    for chunk in (1, 4):
        on = _decoder(cfg, w, max_num_batched_tokens=4, max_num_batched_requests=1, max_seq_length=max_seq, page_size=16, kernel_mode="online")
        on.meta["tokens"].copy_(ref_tokens.cuda())
        on.meta["num_new_tokens"].fill_(chunk)
        on.mpk.init_request_resources()
        # step by step: after each pass the last row's sampled token is the model's choice for the next position.  The
        # offline run ingested the prompt in other chunk sizes (other kernel forms, other fp32 summation orders), so the
        # two are compared where this run's own top-2 margin exceeds 0.05
        it = hits = 0
        while True:
            fin = on.mpk.run_steps(1)
            if fin:
                break
            n = int(on.meta["qo_indptr_buffer"][1].item())
            assert int(on.meta["step"][0].item()) == it * chunk
            pos_next = it * chunk + n
            lg = on.logits()[n - 1].float().cpu()
            tok = int(on.meta["output_tokens"][n - 1, 0].item())
            assert tok == int(lg.argmax())
            top2 = lg.topk(2).values
            if P <= pos_next < max_seq and float(top2[0] - top2[1]) > 0.05:
                assert tok == int(ref[pos_next]), f"chunk {chunk}: token for position {pos_next}"
                hits += 1
            it += 1
            assert it < 100
        assert hits >= (5 if chunk == 1 else 2)
        # the reference's stop rule, on the step value from before the advance (persistent_kernel.cuh:552-565)
        assert int(on.meta["step"][0].item()) >= max_seq - 2
        assert torch.equal(on.meta["tokens"].cpu(), ref_tokens), "online mode must not write tokens"
        on.mpk.finalize()


def test_online_notoken_rejects_a_batch_it_cannot_run():
    """A request with more rows than max_tokens_per_request (or a sequence shorter than its rows, or rows that overlap)
    is not truncated: the launch runs nothing, mk_wait reports MK_EINVAL, and the K/V cache is untouched."""
    from mirage import _capi
    from oracle.qwen3_ref import make_model_weights
    cfg = _cfg()
    w = make_model_weights(cfg, seed=43)
    R, B, max_seq, PS = 3, 16, 48, 16
    on = _decoder(cfg, w, max_num_batched_tokens=B, max_num_batched_requests=R, max_seq_length=max_seq, page_size=PS, total_requests=R,
                  kernel_mode="online_notoken")  # max_tokens_per_request defaults to 8
    m = on.meta

    def describe(qo, kv_ptr, last):
        m["input_tokens"].copy_(torch.arange(B, dtype=torch.int64).view(-1, 1) % cfg.vocab_size)
        m["qo_indptr_buffer"].copy_(torch.tensor(qo, dtype=torch.int32))
        m["paged_kv_indptr_buffer"].copy_(torch.tensor(kv_ptr, dtype=torch.int32))
        m["paged_kv_indices_buffer"].copy_(torch.arange(m["paged_kv_indices_buffer"].numel(), dtype=torch.int32))
        m["paged_kv_last_page_len_buffer"].copy_(torch.tensor(last, dtype=torch.int32))
        torch.cuda.synchronize()

    caches = [on.k_cache, on.v_cache]
    for c in caches:
        c.fill_(0.25)
    # a valid request (4 rows of a 4-long sequence) next to one with 9 rows: over the cap of 8
    describe([0, 4, 13, 13], [0, 1, 2, 2], [4, 9, 0])
    with pytest.raises(_capi.MkError, match="max_tokens_per_request"):
        on.mpk()
    # a sequence shorter than its new rows (2 positions, 3 rows)
    describe([0, 3, 3, 3], [0, 1, 1, 1], [2, 0, 0])
    with pytest.raises(_capi.MkError, match="shorter than its new rows"):
        on.mpk()
    # rows beyond max_num_batched_tokens
    describe([0, 8, 16, 24], [0, 1, 2, 3], [8, 8, 8])
    with pytest.raises(_capi.MkError, match="rows outside"):
        on.mpk()
    torch.cuda.synchronize()
    assert all(bool((c == 0.25).all()) for c in caches), "a rejected batch must not append K/V rows"
    # the handle stays usable: the same shape of batch within the limits runs
    describe([0, 4, 12, 12], [0, 1, 2, 2], [4, 8, 0])
    on.mpk()
    assert on.mpk.stats()["aborted"] == 0
    assert not all(bool((c == 0.25).all()) for c in caches)
    on.mpk.finalize()
