"""Pins the scheduler oracle (oracle/sched_ref.c, restating persistent_kernel.cuh:380-536) against a hand-simulated
schedule and against invariants every correct continuous-batching scheduler satisfies."""
import numpy as np
import pytest

from oracle.sched_ref import SchedulerOracle


def test_hand_simulated_schedule():
    """3 requests with prompts of 5 / 9 / 2 tokens, 3 batch slots, 4 tokens per iteration, 4-token pages, max_seq 12.
    Expected values below were worked out by hand from the rules: running requests first (prefill chunk = remaining
    prompt capped by 8 and by the free token budget, decode = 1 token), then admissions; pages allocated in ring order."""
    p0, p1, p2 = [1, 2, 3, 4, 5], [11, 12, 13, 14, 15, 16, 17, 18, 19], [21, 22]
    o = SchedulerOracle([p0, p1, p2], max_requests=3, max_tokens=4, max_pages=8, page_size=4, max_seq=12)
    # iteration 1: request 0 gets the whole budget (4 of its 5 prompt tokens), one page
    assert o.step() == 4
    assert o["request_ids"].tolist() == [0, -1, -1]
    assert o["qo_indptr"].tolist() == [0, 4, 4, 4] and o["kv_indptr"].tolist() == [0, 1, 1, 1]
    assert o["kv_indices"][:1].tolist() == [0] and o["kv_last_page_len"][0] == 4
    assert o["input_tokens"].tolist() == [1, 2, 3, 4]
    # iteration 2: request 0 feeds its last prompt token (position 4 -> second page), request 1 is admitted with 3 tokens
    assert o.step([100, 101, 102, 103]) == 4
    assert o["step"].tolist() == [4, 0, 0]
    assert o["request_ids"].tolist() == [0, 1, -1]
    assert o["qo_indptr"].tolist() == [0, 1, 4, 4] and o["kv_indptr"].tolist() == [0, 2, 3, 3]
    assert o["kv_indices"][:3].tolist() == [0, 1, 2] and o["kv_last_page_len"][:2].tolist() == [1, 3]
    assert o["input_tokens"].tolist() == [5, 11, 12, 13]
    assert o["tokens"][0, 5] == 0  # outputs of prompt positions are not committed
    # iteration 3: request 0's first generated token (output row 0 of the previous batch) is committed at position 5 and fed
    assert o.step([120, 121, 122, 123]) == 4
    assert o["step"].tolist() == [5, 3, 0]
    assert o["tokens"][0, 5] == 120 and o["tokens"][1, 9] == 0
    assert o["input_tokens"].tolist() == [120, 14, 15, 16]
    assert o["qo_indptr"].tolist() == [0, 1, 4, 4] and o["kv_indptr"].tolist() == [0, 2, 4, 4]
    assert o["kv_indices"][:4].tolist() == [0, 1, 2, 3] and o["kv_last_page_len"][:2].tolist() == [2, 2]
    # iteration 4: request 1 still has 3 prompt tokens; no room for request 2 (budget exhausted)
    assert o.step([130, 131, 132, 133]) == 4
    assert o["input_tokens"].tolist() == [130, 17, 18, 19] and o["request_ids"].tolist() == [0, 1, -1]
    assert o["kv_indptr"].tolist() == [0, 2, 5, 5] and o["kv_indices"][:5].tolist() == [0, 1, 2, 3, 4]
    # iteration 5: both decode (1 token each), request 2 is admitted with its 2 prompt tokens
    assert o.step([140, 141, 142, 143]) == 4
    assert o["request_ids"].tolist() == [0, 1, 2]
    assert o["input_tokens"].tolist() == [140, 143, 21, 22]  # request 1's first generated token is output row 3 (its last prompt row)
    assert o["qo_indptr"].tolist() == [0, 1, 2, 4] and o["kv_indptr"].tolist() == [0, 2, 5, 6]
    assert o["step"].tolist() == [7, 9, 0]


@pytest.mark.parametrize("R,B,PS,max_seq,n_req,seed", [(3, 4, 4, 12, 3, 0), (4, 16, 8, 40, 9, 1), (8, 8, 16, 33, 20, 2), (2, 1, 4, 10, 3, 3),
                                                         (64, 64, 4096, 50, 64, 4)])
def test_scheduler_invariants(R, B, PS, max_seq, n_req, seed):
    rng = np.random.default_rng(seed)
    prompts = [list(rng.integers(1, 1000, size=int(rng.integers(1, max_seq - 2)))) for _ in range(n_req)]
    pages_per_req = (max_seq + PS - 1) // PS
    max_pages = R * pages_per_req
    eos = 777
    o = SchedulerOracle(prompts, R, B, max_pages, PS, max_seq, eos=eos)
    fed = [[] for _ in range(n_req)]
    it = 0
    while True:
        out = rng.integers(1000, 2000, size=B)
        if it % 7 == 3:
            out[int(rng.integers(0, B))] = eos  # occasionally an EOS is sampled
        n = o.step(out if it else None)
        if n == 0:
            break
        it += 1
        assert it < 20000
        qo, kvp, ids = o["qo_indptr"], o["kv_indptr"], o["request_ids"]
        assert n <= B and qo[R] == n
        active = [i for i in range(R) if ids[i] >= 0]
        assert active == list(range(len(active))), "active slots are compacted to the front"
        owned = []
        for i in active:
            req = int(ids[i])
            cnt = qo[i + 1] - qo[i]
            st = int(o["step"][req])
            assert 0 <= cnt <= 8
            if st >= len(prompts[req]):
                assert cnt <= 1, "decode feeds at most one token"
            toks = o["input_tokens"][qo[i]:qo[i + 1]].tolist()
            assert toks == o["tokens"][req, st:st + cnt].tolist()
            fed[req].extend(toks)
            npg = kvp[i + 1] - kvp[i]
            assert npg == (st + cnt + PS - 1) // PS, "a request owns exactly the pages its tokens need"
            last = (st + cnt) % PS
            assert o["kv_last_page_len"][i] == (PS if last == 0 else last)
            owned += o["kv_indices"][kvp[i]:kvp[i + 1]].tolist()
        assert len(owned) == len(set(owned)), "no page is owned twice"
        assert len(owned) + o.free_pages == max_pages, "pages are conserved"
    for req in range(n_req):
        P = len(prompts[req])
        assert fed[req][:P] == prompts[req], "every prompt token is fed exactly once, in order"
        final = int(o["step"][req])
        row = o["tokens"][req]
        assert fed[req] == row[:len(fed[req])].tolist()
        stopped_by_eos = final >= P and row[final] == eos
        assert stopped_by_eos or final + 1 >= max_seq, "a request ends at EOS (after its prompt) or when the sequence is full"
    assert o.free_pages == max_pages, "all pages are back in the ring"
