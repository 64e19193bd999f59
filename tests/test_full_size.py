"""Full-size checks of the headline configurations (36-layer Qwen3-8B shape, vocab 151,936; 48-layer Qwen3-30B-A3B shape).

* configuration 3 (BS=1): the 80-token prompt and the first decode steps are teacher-forced through the kernel-order
  CPU oracle with the SAME weights (generated on the GPU, copied to the host).  This is the only place where the
  151,936-row LM head, the argmax over it and the full depth are asserted (reference driver: demo/qwen3/demo.py:1134-1230);
  see the test's docstring for what can and what cannot hold at 36 layers.
* configurations 4 and 5 at their full step counts: size-independent properties -- two runs give bit-identical tokens,
  one persistent launch equals a run cut into many launches, and the scheduler's end state (iterations, step[], page
  tables) is what the C restatement of the reference scheduler predicts (persistent_kernel.cuh:380-536).
"""
import time

import pytest
import torch

pytestmark = pytest.mark.gpu


def _say(capsys, msg):
    with capsys.disabled():
        print(f"\n    [{time.strftime('%H:%M:%S')}] {msg}", end="", flush=True)


def _weights_to_host(w):
    return {"embed": w["embed"].cpu(), "layers": [{k: v.cpu() for k, v in lw.items()} for lw in w["layers"]],
            "final_norm": w["final_norm"].cpu(), "lm_head": w["lm_head"].cpu()}


def test_config3_full_size_teacher_forced(capsys):
    """What holds at full depth, and why the per-logit tolerance of the small-model tests does not: a random-init 36-layer
    model amplifies a one-ulp difference in a hidden state by about 10 % per layer, so two evaluations that round at
    the same points and differ ONLY in summation order (the oracle with fp32 sums and the oracle with float64 sums) end
    3 % apart in the final hidden state and up to 0.23 apart in single logits.  The GPU is a third such evaluation.
    Asserted here, teacher-forced over the 80-token prompt and the first decode steps:
    (1) the LM head (151,936 rows) and the argmax are exact on the GPU's OWN final hidden state: logits within 1 bf16
        ulp of the fp32-accumulate oracle head, sampled token = lowest index of the maximum of the GPU's logits;
    (2) end to end the GPU is no further from the float64-sum oracle than 1.5 x the distance between the two oracles
        (max |diff| and relative L2 of the logits), and its logits have cosine > 0.999 with it;
    (3) the sampled token's logit in the float64-sum oracle is within twice the largest single-logit distance between the
        two oracles of that oracle's maximum, and it IS that oracle's argmax wherever the top-2 margin exceeds that bound.
    (2) and (3) are asserted on EVERY row the run produces -- all 80 prompt positions (teacher-forced by construction:
    the kernel samples a token for every prompt row, the scheduler only does not use it) and the decode rows -- so that
    the argmax comparison is made on the rows whose margin is decisive: at least eight of them."""
    from demo_qwen3 import Qwen3Decoder, Qwen3Shape, random_weights
    from helpers import bf16_ulp_diff
    from oracle.qwen3_ref import KVCache, Qwen3Config, Qwen3Oracle, argmax_k, linear_k
    torch.set_num_threads(16)
    shape = Qwen3Shape()  # 36 layers, hidden 4096, 32 q / 8 kv heads, intermediate 12288, vocab 151936
    cfg = Qwen3Config()
    assert (cfg.num_layers, cfg.vocab_size, cfg.hidden_size) == (shape.num_layers, shape.vocab_size, shape.hidden_size) == (36, 151936, 4096)
    P, NEW, max_seq = 80, 3, 1200
    _say(capsys, "generating 8B random weights on the GPU")
    wg = random_weights(shape, seed=0)
    dec = Qwen3Decoder(shape, wg, max_num_batched_tokens=8, max_num_batched_requests=1, max_seq_length=max_seq, page_size=4096)
    prompt = torch.randint(0, shape.vocab_size, (P,), generator=torch.Generator().manual_seed(0))
    dec.load_prompts([prompt])
    # GPU: prompt in chunks of 8 tokens, then NEW decode steps; keep the logits and the sampled token of every row, and the
    # final normalised hidden state of the prompt's last token (an 8-row iteration) and of every decode step (1-row iterations)
    gpu_logits, gpu_hidden, gpu_tokens = [], [], []
    for it in range(P // 8 + NEW):
        assert not dec.mpk.run_steps(1)
        rows = range(8) if it < P // 8 else range(1)
        lg, hd, tk = dec.logits().cpu(), dec.t["rmsnorm_out"].to_torch().cpu(), dec.meta["output_tokens"][:, 0].cpu()
        for r in rows:
            gpu_logits.append(lg[r].clone())
            gpu_hidden.append(hd[r].clone())
            gpu_tokens.append(int(tk[r]))
    n_rows = P + NEW
    assert len(gpu_tokens) == n_rows
    # step[] and tokens[] are committed by the scheduler step that opens the NEXT iteration: the last sampled token is still pending
    assert int(dec.meta["step"][0].item()) == P + NEW - 1
    assert dec.meta["tokens"][0, P:P + NEW].cpu().tolist() == gpu_tokens[P - 1:P - 1 + NEW]
    assert dec.mpk.stats()["aborted"] == 0
    _say(capsys, "copying the weights to the host")
    w = _weights_to_host(wg)
    dec.mpk.finalize()
    del dec, wg
    torch.cuda.empty_cache()
    # (1) head + argmax on the GPU's own hidden state: the last prompt row and the decode rows (and the first prompt row)
    for i in [0] + list(range(P - 1, n_rows)):
        head = linear_k(gpu_hidden[i][None], w["lm_head"])[0]
        ulp, mabs = bf16_ulp_diff(gpu_logits[i], head, floor=1.0 / 16)
        frac = float((gpu_logits[i].float() != head.float()).float().mean())
        assert ulp <= 1.0 and frac < 0.02, f"row {i}: LM head differs from the oracle on the same input: {frac:.4f} of 151936 logits, max {ulp} ulp ({mabs})"
    for i in range(n_rows):
        assert gpu_tokens[i] == int(argmax_k(gpu_logits[i][None])[0]), f"row {i}: sampled token is not the lowest index of the maximum logit"
    _say(capsys, "LM head and argmax exact on the GPU's own hidden state; oracles: 80-token prompt (fp32 sums, then float64 sums)")
    o32, o64 = Qwen3Oracle(cfg, w, "kernel"), Qwen3Oracle(cfg, w, "kernel", acc=torch.float64)
    c32, c64 = KVCache(cfg, P + NEW + 2), KVCache(cfg, P + NEW + 2)
    A = o32.forward(prompt, c32, 0)
    B = o64.forward(prompt, c64, 0)
    hits, worst = 0, (0.0, 0.0, 1.0)
    for i in range(n_rows):
        if i >= P:  # decode rows: one more oracle step each, fed with the token the GPU sampled
            ids = torch.tensor([gpu_tokens[i - 1]])
            a = o32.forward(ids, c32, i)[0].double()
            b = o64.forward(ids, c64, i)[0].double()
        else:
            a, b = A[i].double(), B[i].double()
        g = gpu_logits[i].double()
        d_or, d_gpu = (a - b).abs(), (g - b).abs()
        rel = lambda d: float(d.norm() / b.norm())
        cos = float(torch.nn.functional.cosine_similarity(g, b, dim=0))
        if i >= P - 1:
            within = float((d_gpu <= 2e-2 + 1e-2 * b.abs()).double().mean())
            _say(capsys, f"row {i}: oracle fp32 vs float64 sums max |diff| {float(d_or.max()):.3f} rel L2 {rel(d_or):.4f}; GPU vs float64-sum oracle "
                         f"max |diff| {float(d_gpu.max()):.3f} rel L2 {rel(d_gpu):.4f} cosine {cos:.5f} ({within:.2f} of logits within 2e-2 / 1e-2)")
        worst = (max(worst[0], float(d_gpu.max()) / max(float(d_or.max()), 1e-3)), max(worst[1], rel(d_gpu) / max(rel(d_or), 1e-4)), min(worst[2], cos))
        assert float(d_gpu.max()) <= 1.5 * float(d_or.max()) + 1e-2, f"row {i}: GPU is further from the oracle than summation order explains"
        assert rel(d_gpu) <= 1.5 * rel(d_or) + 1e-3 and cos > 0.999
        # the sampled token is a near-maximal token of the oracle: its oracle logit is within the drift of the oracle's maximum
        assert float(b.max() - b[gpu_tokens[i]]) <= 2 * float(d_or.max()), f"row {i}: the GPU sampled a token the oracle ranks far from the top"
        top2 = b.topk(2).values
        if float(top2[0] - top2[1]) > 2 * float(d_or.max()):
            assert gpu_tokens[i] == int(b.argmax()), f"row {i}: argmax differs from the oracle at a margin of {float(top2[0] - top2[1]):.3f}"
            hits += 1
    _say(capsys, f"done: {n_rows} rows checked (worst GPU/oracle distance ratio: max |diff| {worst[0]:.2f}, rel L2 {worst[1]:.2f}; lowest cosine {worst[2]:.5f}), "
                 f"{hits} with a decisive margin\n")
    assert hits >= 8, f"only {hits} rows had a top-2 margin above the oracle's own drift: the argmax comparison needs more rows"


def _sched_oracle_end_state(prompt_lens, R, B, max_pages, page_size, max_seq):
    """Run the C restatement of the reference scheduler to the end (token values do not matter with EOS disabled)."""
    from oracle.sched_ref import SchedulerOracle
    orc = SchedulerOracle([[1] * n for n in prompt_lens], R, B, max_pages, page_size, max_seq)
    iters = 0
    while orc.step([1] * B) > 0:
        iters += 1
        assert iters < 100000
    return orc, iters


def _property_run(capsys, shape, B, P, new_tokens, chunk):
    from demo_qwen3 import Qwen3Decoder, random_weights
    max_seq = P + new_tokens + 1
    _say(capsys, f"generating weights ({shape.num_layers} layers)")
    w = random_weights(shape, seed=0)
    dec = Qwen3Decoder(shape, w, max_num_batched_tokens=B, max_num_batched_requests=B, max_seq_length=max_seq, page_size=4096)
    prompts = [torch.randint(0, shape.vocab_size, (P,), generator=torch.Generator().manual_seed(r)) for r in range(B)]
    _say(capsys, "run 1: one persistent launch")
    t1, s1 = dec.generate(prompts)
    it1 = dec.mpk.stats()["iterations"]
    meta1 = {k: v.clone() for k, v in dec.meta.items()}
    _say(capsys, f"run 1 took {dec.mpk.stats()['last_launch_ms']:.0f} ms for {it1} iterations; run 2: launches of {chunk} iterations")
    dec.load_prompts(prompts)
    n_launch = 0
    while not dec.mpk.run_steps(chunk):
        n_launch += 1
        if n_launch % 64 == 0:
            _say(capsys, f"  {n_launch} launches")
    t2 = dec.meta["tokens"].cpu()
    assert dec.mpk.stats()["iterations"] == it1
    assert dec.mpk.stats()["aborted"] == 0
    # determinism / single launch == many launches: the first differing position is reported
    if not torch.equal(t1, t2):
        bad = (t1 != t2).nonzero()[0].tolist()
        raise AssertionError(f"tokens differ between the two runs, first at request {bad[0]} position {bad[1]}: {int(t1[bad[0], bad[1]])} vs {int(t2[bad[0], bad[1]])}")
    assert all(int(s) == max_seq - 1 for s in s1)
    assert bool((t1[:, P:max_seq] >= 0).all()) and bool((t1[:, P:max_seq] < shape.vocab_size).all())
    for r in range(B):
        assert t1[r, :P].tolist() == prompts[r].tolist()
    # end state of the scheduler as the C oracle predicts it
    ref, iters = _sched_oracle_end_state([P] * B, B, B, dec.max_pages, 4096, max_seq)
    assert it1 == iters, f"{it1} iterations on the GPU, the scheduler oracle predicts {iters}"
    for name, key in (("step", "step"), ("qo_indptr", "qo_indptr_buffer"), ("kv_indptr", "paged_kv_indptr_buffer")):
        assert dec.meta[key].cpu().tolist() == ref[name].tolist(), name
    for k in ("step", "qo_indptr_buffer", "paged_kv_indptr_buffer", "paged_kv_indices_buffer", "paged_kv_last_page_len_buffer"):
        assert torch.equal(meta1[k], dec.meta[k]), f"{k} differs between the two runs"
    dec.mpk.finalize()
    _say(capsys, "done\n")


@pytest.mark.parametrize("B", [32, 64])
def test_config4_full_size_properties(capsys, B):
    """36-layer Qwen3-8B shape, B independent 80-token prompts, 1024 new tokens each."""
    from demo_qwen3 import Qwen3Shape
    _property_run(capsys, Qwen3Shape(), B, 80, 1024, chunk=37)


@pytest.mark.parametrize("B", [1, 32])
def test_config5_full_size_properties(capsys, B):
    """48-layer Qwen3-30B-A3B shape (128 experts, top-8), 80-token prompts, 512 new tokens."""
    from demo_qwen3 import Qwen3Shape
    _property_run(capsys, Qwen3Shape.qwen3_30b_a3b(48), B, 80, 512, chunk=29)


def test_config4_full_size_bs8_several_pages_per_request(capsys):
    """36-layer Qwen3-8B shape at B=8: the same generation with one 4096-position page per request and with 64-position
    pages (six to seven per request, handed out by the on-GPU scheduler as the contexts grow, so the requests' pages
    interleave) gives the same tokens -- where a K/V row lives must not matter -- and the page tables end as the C
    restatement of the scheduler predicts."""
    from demo_qwen3 import Qwen3Decoder, Qwen3Shape, random_weights
    shape, B, P, new_tokens = Qwen3Shape(), 8, 80, 320
    max_seq = P + new_tokens + 1
    _say(capsys, "generating weights (36 layers)")
    w = random_weights(shape, seed=0)
    prompts = [torch.randint(0, shape.vocab_size, (P,), generator=torch.Generator().manual_seed(r)) for r in range(B)]
    runs = {}
    for ps in (4096, 64):
        dec = Qwen3Decoder(shape, w, max_num_batched_tokens=B, max_num_batched_requests=B, max_seq_length=max_seq, page_size=ps)
        _say(capsys, f"page_size {ps}: one persistent launch")
        toks, steps = dec.generate(prompts)
        st = dec.mpk.stats()
        assert st["aborted"] == 0 and all(int(s) == max_seq - 1 for s in steps)
        ref, iters = _sched_oracle_end_state([P] * B, B, B, dec.max_pages, ps, max_seq)
        assert st["iterations"] == iters
        for name, key in (("step", "step"), ("qo_indptr", "qo_indptr_buffer"), ("kv_indptr", "paged_kv_indptr_buffer")):
            assert dec.meta[key].cpu().tolist() == ref[name].tolist(), (ps, name)
        runs[ps] = toks
        dec.mpk.finalize()
    if not torch.equal(runs[4096], runs[64]):
        bad = (runs[4096] != runs[64]).nonzero()[0].tolist()
        raise AssertionError(f"tokens depend on the page size, first at request {bad[0]} position {bad[1]}")
    _say(capsys, "done\n")
