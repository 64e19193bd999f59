"""The kernel's on-GPU scheduler against the C scheduler oracle: after every iteration the meta tensors must be
bit-identical (integer work).  The model is tiny; only the scheduling state is compared."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,R,total,page_size,max_seq,eos_every", [(4, 3, 3, 4, 12, 0), (8, 4, 9, 8, 24, 0), (16, 16, 20, 16, 30, 5), (1, 1, 2, 4, 9, 0)])
def test_meta_tensors_match_scheduler_oracle(B, R, total, page_size, max_seq, eos_every):
    from demo_qwen3 import Qwen3Decoder, Qwen3Shape, random_weights
    from oracle.sched_ref import SchedulerOracle
    shape = Qwen3Shape(hidden_size=1024, num_q_heads=8, num_kv_heads=2, head_dim=128, intermediate_size=512, num_layers=1, vocab_size=512)
    w = random_weights(shape, seed=1)
    rng = np.random.default_rng(B * 100 + total)
    prompts = [torch.from_numpy(rng.integers(0, shape.vocab_size, size=int(rng.integers(1, max_seq - 3)))) for _ in range(total)]
    pages = R * ((max_seq + page_size - 1) // page_size)
    eos = 0x7FFFFFFF
    dec = Qwen3Decoder(shape, w, max_num_batched_tokens=B, max_num_batched_requests=R, max_seq_length=max_seq, page_size=page_size,
                       max_num_pages=pages, total_requests=total, eos_token_id=eos)
    if eos_every:
        # pick an EOS id the model actually emits: run once, take a frequently generated token
        toks, _ = dec.generate(prompts)
        gen = torch.cat([toks[r, len(prompts[r]):] for r in range(total)])
        eos = int(gen[gen > 0].mode().values)
        dec.mpk.finalize()
        dec = Qwen3Decoder(shape, w, max_num_batched_tokens=B, max_num_batched_requests=R, max_seq_length=max_seq, page_size=page_size,
                           max_num_pages=pages, total_requests=total, eos_token_id=eos)
    dec.load_prompts(prompts)
    orc = SchedulerOracle([p.tolist() for p in prompts], R, B, pages, page_size, max_seq, eos=eos)
    names = {"step": "step", "input_tokens": "input_tokens", "qo_indptr_buffer": "qo_indptr", "paged_kv_indptr_buffer": "kv_indptr",
             "paged_kv_last_page_len_buffer": "kv_last_page_len"}
    it = 0
    out_prev = None
    while True:
        n = orc.step(out_prev)
        fin = dec.mpk.run_steps(1)
        if n == 0:
            assert fin, "the kernel must report completion when the oracle schedules nothing"
            break
        assert not fin
        it += 1
        assert it < 5000
        nreq = int((orc["request_ids"] >= 0).sum())
        for gk, ok in names.items():
            got = dec.meta[gk].cpu().numpy().reshape(-1)
            exp = orc[ok].reshape(-1)
            m = {"input_tokens": n, "paged_kv_last_page_len_buffer": nreq}.get(gk, len(exp))
            assert np.array_equal(got[:m], exp[:m]), f"iteration {it}: {gk} differs: {got[:m]} vs {exp[:m]}"
        npg = int(orc["kv_indptr"][R])
        assert np.array_equal(dec.meta["paged_kv_indices_buffer"].cpu().numpy()[:npg], orc["kv_indices"][:npg])
        out_prev = dec.meta["output_tokens"].cpu().numpy().reshape(-1)
    assert np.array_equal(dec.meta["tokens"].cpu().numpy(), orc["tokens"])
    assert np.array_equal(dec.meta["step"].cpu().numpy(), orc["step"])
    dec.mpk.finalize()
