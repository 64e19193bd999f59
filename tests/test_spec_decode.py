"""Prompt-lookup speculative decoding: the reference's three integer tasks (tasks/speculative_decoding/prompt_lookup.cuh,
target_verify.cuh) -- CPU oracle pinned on the reference's own test scenarios and on brute force, host lowering, and on
the GPU the stages bit for bit against the oracle in every iteration plus the property that greedy speculative decoding
reproduces plain greedy decoding."""
import random

import pytest
import torch

from oracle.spec_ref import (LLONG_MAX, accepted_with_eos, find_ngram_global, find_ngram_partial, prompt_lookup_rows,
                             speculative_greedy_decode, target_verify_greedy)


# ----------------------------------------------------------------------------- oracle pins (CPU)
def test_oracle_reference_test_scenarios():
    """tests/runtime_python/test_prompt_lookup.py of the reference: a planted n-gram at 100 with five planted followers,
    the same n-gram closing the 515-token prompt -> [regular token, followers]; no earlier occurrence -> -1s.  (That test
    hands the partial task input_token_num = PROMPT_LEN and the global task step = PROMPT_LEN.)"""
    g = torch.Generator().manual_seed(0)
    N, L, PROMPT_LEN = 3, 5, 515
    toks = torch.randint(40, 1000, (2048,), generator=g).tolist()
    toks[100:103] = [10, 20, 30]
    toks[103:108] = [4, 5, 6, 7, 8]
    toks[PROMPT_LEN - 3:PROMPT_LEN] = [10, 20, 30]
    toks[PROMPT_LEN] = 99
    part = find_ngram_partial(toks, PROMPT_LEN, N, 96)
    assert min(part) == 100 and part[0] == 100 and sum(p != LLONG_MAX for p in part) == 1  # idx 100 is in task (100 // 128) % 96 = 0
    assert find_ngram_global(part, toks, PROMPT_LEN, N, L) == [99, 4, 5, 6, 7, 8]
    toks2 = torch.randint(40, 1000, (2048,), generator=g).tolist()
    toks2[PROMPT_LEN - 3:PROMPT_LEN] = [10, 20, 30]
    toks2[PROMPT_LEN] = 99
    part2 = find_ngram_partial(toks2, PROMPT_LEN, N, 96)
    assert all(p == LLONG_MAX for p in part2)
    assert find_ngram_global(part2, toks2, PROMPT_LEN, N, L) == [99, -1, -1, -1, -1, -1]


def _brute_first(tokens, T, N):
    """Earliest idx in [0, T - N) with tokens[idx:idx+N] == tokens[T-N:T], or None."""
    tail = tokens[T - N:T]
    for idx in range(0, T - N):
        if tokens[idx:idx + N] == tail:
            return idx
    return None


@pytest.mark.parametrize("N,L,P", [(3, 5, 96), (2, 4, 7), (1, 3, 3), (4, 7, 96)])
def test_oracle_against_brute_force(N, L, P):
    rnd = random.Random(N * 100 + L)
    for trial in range(60):
        T = rnd.randint(1, 700)
        toks = [rnd.randint(0, 3) for _ in range(T + L + 4)]  # tiny vocabulary: matches everywhere, also overlapping the tail
        part = find_ngram_partial(toks, T, N, P)
        first = _brute_first(toks, T, N) if T > N else None
        assert (min(part) if min(part) != LLONG_MAX else None) == first
        for k, p in enumerate(part):  # every task holds the earliest match of ITS share
            if p != LLONG_MAX:
                assert (p // 128) % P == k and toks[p:p + N] == toks[T - N:T]
        step = T - 1
        rows = find_ngram_global(part, toks, step, N, L)
        want = [toks[step]] + [(toks[first + N + t] if first is not None and first + N + t <= step else -1) for t in range(L)]
        assert rows == want


def test_oracle_verify_cases():
    # the reference's semantics: spec[0] is the real token, spec[1 + i] is compared with target[i]
    assert target_verify_greedy([7, 1, 2, 3], [1, 2, 3, 9], 3) == (4, [1, 2, 3, 9])   # all guesses right: all four targets are new tokens
    assert target_verify_greedy([7, 1, 2, 3], [1, 5, 3, 9], 3) == (2, [1, 5])        # second guess wrong: its own target still counts
    assert target_verify_greedy([7, -1, -1, -1], [4, 5, 6, 7], 3) == (1, [4])        # no guesses: plain decoding
    assert target_verify_greedy([7, 4, -1, -1], [4, 5, 6, 7], 3) == (2, [4, 5])
    assert accepted_with_eos([7, 1, 2, 3], [1, 2, 3, 9], eos_token_id=2) == 2        # cut behind the accepted EOS
    assert accepted_with_eos([7, 1, 2, 3], [1, 5, 2, 9], eos_token_id=2) == 2        # an EOS behind a wrong guess is not reached


def test_oracle_speculative_equals_plain_greedy():
    """For any deterministic next-token function the accepted tokens are exactly the tokens plain greedy decoding emits."""
    def model(prefix):  # a little hash machine that falls into loops, so that n-grams recur
        return (prefix[-1] * 7 + prefix[-2] * 3 + len(prefix) % 2) % 11 if len(prefix) > 1 else 1
    for seed in range(5):
        rnd = random.Random(seed)
        prompt = [rnd.randint(0, 10) for _ in range(rnd.randint(4, 30))]
        plain = list(prompt)
        while len(plain) < 120:
            plain.append(model(plain))
        spec, iters = speculative_greedy_decode(model, prompt, 120, ngram_size=2, spec_length=4)
        assert spec == plain
        assert iters < 120 - len(prompt)  # some guesses were accepted


# ----------------------------------------------------------------------------- front end and lowering (CPU)
def test_spec_decode_class_and_lowering():
    import mirage as mi
    from mirage.mpk.speculative import LookaheadConfig, PromptLookupConfig
    cfg = mi.mpk.spec_decode_class("promptlookup", ngram_size=3, spec_length=5)
    assert isinstance(cfg, PromptLookupConfig) and (cfg.method, cfg.ngram_size, cfg.spec_length) == ("promptlookup", 3, 5)
    assert isinstance(mi.mpk.spec_decode_class("lookahead", 3, 7), LookaheadConfig) and mi.mpk.spec_decode_class(None, 3, 5) is None
    with pytest.raises(NotImplementedError):
        mi.mpk.spec_decode_class("medusa", 3, 5)


def _host_graph(spec, B=8, R=2, max_seq=64):
    import mirage as mi
    from helpers import make_meta
    meta = make_meta(R, max_seq, B, R, 8, device="cpu")
    mpk = mi.PersistentKernel(mode="offline", world_size=1, mpi_rank=0, num_workers=256, num_local_schedulers=0, num_remote_schedulers=0,
                              max_seq_length=max_seq, max_num_batched_requests=R, max_num_batched_tokens=B, max_num_pages=8, page_size=16,
                              meta_tensors=meta, profiler_tensor=None, trace_name=None, spec_decode_config=spec, use_cutlass_kernel=False, eos_token_id=2)
    return mpk, meta


def test_lowering_of_the_three_tasks():
    """Host only (no device): the n-gram pair in front of the embedding, the verify task behind the sampling stages."""
    import mirage as mi
    spec = mi.mpk.spec_decode_class("promptlookup", ngram_size=3, spec_length=5)
    mpk, meta = _host_graph(spec)
    tokens = mpk.attach_input(meta["tokens"], "all_tokens")
    ids = mpk.draft_forward_layer_dispatcher(spec_decode_config=spec, tokens=tokens, grid_dim=(96, 1, 1), block_dim=(128, 1, 1))
    assert (ids.dim(0), ids.dim(1)) == (2, 6)  # the reference's [requests, spec_length + 1]: 12 >= the 8 rows of an iteration
    emb = mpk.attach_input(torch.zeros(64, 256, dtype=torch.bfloat16), "embed_tokens")
    x = mpk.new_tensor(dims=(8, 256), dtype=mi.bfloat16, name="embed_out", io_category="cuda_tensor")
    mpk.embed_layer(input=ids, weight=emb, output=x, grid_dim=(1, 1, 1), block_dim=(128, 1, 1), input_source=1)
    logits = mpk.new_tensor(dims=(8, 64), dtype=mi.bfloat16, name="argmax_in", io_category="cuda_tensor")
    head = mpk.attach_input(torch.zeros(64, 256, dtype=torch.bfloat16), "lm_head")
    mpk.linear_layer(input=x, weight=head, output=logits, grid_dim=(4, 1, 1), block_dim=(128, 1, 1))
    out = mpk.attach_input(meta["output_tokens"], "output_token")
    mpk.argmax_layer(input=logits, output=out, grid_dim=(1, 1, 1), block_dim=(128, 1, 1))
    v = mpk.verify_layer_dispatcher(spec_decode_config=spec, spec_tokens=ids, target_output=out)
    assert (v.dim(0), v.dim(1)) == (1, 1)
    prog = [l.split()[1] for l in mpk.describe_program().splitlines()]
    assert prog == ["NGRAM_PARTIAL", "NGRAM_GLOBAL", "EMBED", "LINEAR", "ARGMAX_PARTIAL", "ARGMAX_REDUCE", "VERIFY"]
    assert "ngram=3 tasks=96" in mpk.describe_program() and "ngram=3 spec=5" in mpk.describe_program()
    tg = mpk.kn_graph.generate_task_graph(1, 0)["json_file"]
    assert '"task_type": 112' in tg and '"task_type": 113' in tg and '"task_type": 114' in tg  # runtime_header.h:106-108
    # the search runs over the `tokens` meta tensor and nothing else
    mpk2, meta2 = _host_graph(spec)
    other = mpk2.attach_input(torch.zeros(2, 64, dtype=torch.int64), "not_the_tokens")
    mpk2.draft_forward_layer_dispatcher(spec_decode_config=spec, tokens=other, grid_dim=(96, 1, 1), block_dim=(128, 1, 1))
    with pytest.raises(RuntimeError, match="tokens. meta tensor"):
        mpk2.describe_program()
    # a verify task needs the n-gram tasks that size the token groups
    mpk3, meta3 = _host_graph(spec)
    a = mpk3.attach_input(torch.zeros(8, 1, dtype=torch.int64), "a")
    b = mpk3.attach_input(meta3["output_tokens"], "output_token")
    mpk3.verify_layer_dispatcher(spec_decode_config=spec, spec_tokens=a, target_output=b)
    with pytest.raises(RuntimeError, match="find_ngram_global"):
        mpk3.describe_program()


# ----------------------------------------------------------------------------- GPU
def _spec_decoder(cfg, w, spec, n_req, max_seq, **kw):
    from test_qwen3_decode import _decoder
    L1 = spec.spec_length + 1 if spec is not None else 1
    return _decoder(cfg, w, max_num_batched_tokens=max(8, n_req * L1), max_num_batched_requests=n_req, max_seq_length=max_seq, page_size=16,
                    max_tokens_per_request=max(8, L1), spec_decode_config=spec, **kw)


def _prompts(cfg, n_req):
    """Prompts with repeated stretches, so that the n-gram search has something to find from the first decode step on."""
    out = []
    for r in range(n_req):
        g = torch.Generator().manual_seed(100 + r)
        base = torch.randint(1, cfg.vocab_size, (7 + r,), generator=g)
        out.append(torch.cat([base, base[: 4 + r], base[2:6]]))
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("n_req", [1, 3])
def test_stages_match_oracle_every_iteration(n_req):
    import mirage as mi
    from oracle.qwen3_ref import make_model_weights
    from test_qwen3_decode import _small_cfg
    cfg = _small_cfg()
    w = make_model_weights(cfg, seed=11)
    spec = mi.mpk.spec_decode_class("promptlookup", ngram_size=2, spec_length=4)
    max_seq = 96
    dec = _spec_decoder(cfg, w, spec, n_req, max_seq)
    prog = dec.mpk.describe_program()
    assert "NGRAM_PARTIAL" in prog and "NGRAM_GLOBAL" in prog and "VERIFY" in prog
    prompts = _prompts(cfg, n_req)
    dec.load_prompts(prompts)
    part_t = next(t for t in dec.mpk._tensors if t.name == "partial_ngram_output")
    N, L = spec.ngram_size, spec.spec_length
    prev = None  # (step, kept, targets) per request of the previous iteration
    multi_accepts = 0
    for it in range(200):
        finished = dec.mpk.run_steps(1)
        step = dec.meta["step"].cpu().tolist()
        tokens = dec.meta["tokens"].cpu()
        qo = dec.meta["qo_indptr_buffer"].cpu().tolist()
        plen = dec.meta["prompt_lengths"].cpu().tolist()
        if prev is not None:  # the scheduler committed what the previous verify stage kept, no more and no less
            for r, (st0, kept, targets) in prev.items():
                assert step[r] == st0 + kept, (it, r, step[r], st0, kept)
                for j in range(kept):  # (sampled tokens of prompt rows are dropped: those positions hold the prompt)
                    if st0 + 1 + j >= plen[r]:
                        assert int(tokens[r, st0 + 1 + j]) == targets[j], (it, r, j)
        if finished:
            break
        spec_rows = dec.t["spec_tokens"].to_torch().cpu().view(-1).tolist()
        targets = dec.meta["output_tokens"].cpu().view(-1).tolist()
        nnew = dec.meta["num_new_tokens"].cpu().tolist()
        inputs = dec.meta["input_tokens"].cpu().view(-1).tolist()
        part = part_t.to_torch().cpu()
        prev = {}
        # batch slots hold the live requests in request order (all were admitted in the first iteration; a request that
        # reached max_seq_length leaves and the slots behind it move up)
        live = [r for r in range(n_req) if step[r] + 1 < max_seq]
        for slot, r in enumerate(live):
            q0, n = qo[slot], qo[slot + 1] - qo[slot]
            if n <= 0:
                continue
            st0 = step[r]
            hist = tokens[r].tolist()
            if st0 >= plen[r]:  # decoding: rows = newest token + guesses
                want_rows, want_part = prompt_lookup_rows(hist, st0, N, L)
                assert 1 <= n <= min(L + 1, max_seq - 1 - st0), (it, r, n, st0)  # (fewer when the iteration's token budget runs out)
                assert spec_rows[q0:q0 + n] == want_rows[:n], (it, r, spec_rows[q0:q0 + n], want_rows)
                if n > 1:
                    assert part[slot].tolist() == want_part
                kept = accepted_with_eos(want_rows[:n], targets[q0:q0 + n], dec.mpk.eos_token_id)
                assert nnew[r] == kept, (it, r, nnew[r], kept)
                multi_accepts += kept > 1
            else:  # prompt chunk: the scheduler's ids pass through
                assert spec_rows[q0:q0 + n] == inputs[q0:q0 + n] == hist[st0:st0 + n]
                kept = n
            prev[r] = (st0, kept, targets[q0:q0 + n])
    else:
        raise AssertionError("generation did not finish")
    assert multi_accepts >= 3, "no guess was ever accepted: the test exercises nothing"
    dec.mpk.finalize()


@pytest.mark.gpu
def test_speculative_generation_equals_plain_greedy():
    import mirage as mi
    from oracle.qwen3_ref import make_model_weights
    from test_qwen3_decode import _small_cfg
    cfg = _small_cfg()
    w = make_model_weights(cfg, seed=11)
    prompts = _prompts(cfg, 2)
    max_seq = 80
    plain = _spec_decoder(cfg, w, None, 2, max_seq)
    t_plain, s_plain = plain.generate(prompts)
    it_plain = plain.mpk.stats()["iterations"]
    plain.mpk.finalize()
    spec = mi.mpk.spec_decode_class("promptlookup", ngram_size=2, spec_length=5)
    sd = _spec_decoder(cfg, w, spec, 2, max_seq)
    t_spec, s_spec = sd.generate(prompts)
    it_spec = sd.mpk.stats()["iterations"]
    sd.mpk.finalize()
    assert s_spec.tolist() == s_plain.tolist() == [max_seq - 1] * 2
    assert torch.equal(t_spec, t_plain)
    assert it_spec < it_plain, (it_spec, it_plain)  # accepted guesses save iterations


@pytest.mark.gpu
def test_mpk_wrapper_with_prompt_lookup():
    """MPKMetadata(spec_decode="promptlookup"): the Qwen3 builder puts the n-gram tasks in front of the embedding and the
    verify task behind the sampling (the reference's builder leaves this as a TODO, models/qwen3/builder.py:719-745); the
    generation equals the wrapper's plain run."""
    from mirage.mpk import MPK
    from oracle.qwen3_ref import make_model_weights
    from test_mpk_builder import _cfg, _load_prompts, _metadata
    cfg = _cfg()
    w = make_model_weights(cfg, seed=62)
    R, total, max_seq, PS = 2, 2, 72, 16
    prompts = _prompts(cfg, 2)
    runs = {}
    for spec in (None, "promptlookup"):
        md = _metadata(cfg, w, "cuda", R=R, T=12, total=total, max_seq=max_seq, PS=PS)
        md.spec_decode, md.ngram_size, md.spec_length = spec, 2, 5
        md.max_tokens_per_request = 8
        mpk = MPK(md)
        mpk.build()
        mpk.compile()
        prog = mpk.persistent_kernel.describe_program()
        assert ("NGRAM_GLOBAL" in prog and "VERIFY" in prog) == (spec is not None)
        _load_prompts(mpk, prompts)
        torch.cuda.synchronize()
        mpk.init_per_request()
        mpk()
        torch.cuda.synchronize()
        runs[spec] = (mpk.tokens.cpu(), mpk.step.cpu(), mpk.persistent_kernel.stats()["iterations"])
        mpk.finalize()
    assert torch.equal(runs[None][0], runs["promptlookup"][0]) and torch.equal(runs[None][1], runs["promptlookup"][1])
    assert runs["promptlookup"][2] < runs[None][2]
