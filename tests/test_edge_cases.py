"""Edge cases the reference's own operator tests exercise, run through the persistent kernel on the GPU:

* embedding: ids below zero give zero rows (tasks/ampere/embedding.cuh:42-72; tests/runtime_python/test_embedding.py:24-29);
* argmax: a planted maximum at the first / last index and on both sides of every workgroup's slice boundary, ties (lowest
  index wins), all-equal rows and rows of the sentinel -5e4, at vocabulary 151,936 for 1 and 64 rows
  (tasks/mi300/argmax_mi300.cuh:92-157; tests/runtime_python/test_argmax.py:18-36);
* attention closed forms through the attention stage: one position => the output is that position's V row; all scores
  equal (q = 0) => the output is the mean of the V rows seen, for the dot-product form (one token) and the matrix-core
  form (a 16-token chunk at full width)."""
import pytest
import torch

from helpers import bf16_ulp_diff, make_meta, make_mpk

pytestmark = pytest.mark.gpu


def test_embedding_negative_ids_give_zero_rows():
    B, V, H = 8, 1000, 4096
    g = torch.Generator().manual_seed(3)
    table = torch.randn(V, H, generator=g).to(torch.bfloat16)
    meta = make_meta(B, 64, B, B, B)
    mpk = make_mpk(meta, 64, B, B, B, 64, mode="onepass")
    ids = mpk.attach_input(meta["input_tokens"], "ids")
    w = mpk.attach_input(table.cuda(), "table")
    out = mpk.new_tensor((B, H), name="out")
    mpk.embed_layer(input=ids, weight=w, output=out, grid_dim=(1, 1, 1), block_dim=(128, 1, 1), input_source=1)
    mpk.compile()
    for M, idv in ((8, [5, -1, 999, 0, -7, 17, -1, 500]), (3, [-1, -1, 42]), (1, [-3]), (1, [998])):
        out.to_torch().fill_(7.0)
        meta["input_tokens"][:M, 0] = torch.tensor(idv, dtype=torch.int64)
        torch.cuda.synchronize()
        mpk.run_once(list(range(M)), [0] * M)
        got = out.to_torch()[:M].cpu()
        want = torch.stack([table[i] if i >= 0 else torch.zeros(H, dtype=torch.bfloat16) for i in idv])
        assert torch.equal(got, want), f"ids {idv}"
        assert bool((out.to_torch()[M:] == 7.0).all()), "rows beyond the iteration's tokens were written"
    assert mpk.stats()["aborted"] == 0
    mpk.finalize()


def _argmax_graph(B, V):
    import mirage as mi
    meta = make_meta(B, 64, B, B, B)
    mpk = make_mpk(meta, 64, B, B, B, 64, mode="onepass")
    logits = torch.zeros(B, V, dtype=torch.bfloat16, device="cuda")
    x = mpk.attach_input(logits, "logits")
    tasks = 256 if V % 256 == 0 else 128
    pv, pi = mpk.new_tensor((B, tasks), name="pv"), mpk.new_tensor((B, tasks), dtype=mi.int64, name="pi")
    out = mpk.attach_input(meta["output_tokens"], "out")
    mpk.argmax_partial_layer(input=x, output=(pv, pi), grid_dim=(tasks, 1, 1), block_dim=(128, 1, 1))
    mpk.argmax_reduce_layer(input=(pv, pi), output=out, grid_dim=(1, 1, 1), block_dim=(128, 1, 1))
    mpk.compile()
    return mpk, meta, logits


@pytest.mark.parametrize("B", [1, 64])
def test_argmax_planted_maxima_ties_and_flat_rows(B):
    from oracle.qwen3_ref import argmax_k
    V = 151936
    mpk, meta, logits = _argmax_graph(B, V)
    G = mpk.stats()["num_workgroups"]
    per = (V + G - 1) // G
    per += per & 1  # each workgroup scans an even-sized slice
    bounds = [k * per for k in range(1, G) if k * per < V]
    plant = [0, V - 1, 1, V - 2] + [b - 1 for b in bounds] + bounds + [b + 1 for b in bounds]
    g = torch.Generator().manual_seed(9)
    base = (torch.randn(V, generator=g) * 1.3).to(torch.bfloat16)

    def run(rows):
        """rows: list of bf16 [V] tensors (at most B); returns the sampled ids."""
        M = len(rows)
        logits[:M].copy_(torch.stack(rows).cuda())
        meta["output_tokens"].fill_(-5)
        torch.cuda.synchronize()
        mpk.run_once(list(range(M)), [0] * M)
        got = meta["output_tokens"][:M, 0].cpu()
        want = argmax_k(torch.stack(rows))
        assert torch.equal(got, want), f"rows {[(int(a), int(b)) for a, b in zip(got, want) if a != b][:8]} (got, want)"
        return got

    # a planted 65504 (and a row where the planted value only just exceeds the background) at every interesting index
    for i0 in range(0, len(plant), B):
        rows = []
        for j, idx in enumerate(plant[i0:i0 + B]):
            r = base.clone()
            r[idx] = 65504.0 if j % 2 == 0 else float(base.float().max()) + 0.25
            rows.append(r)
        got = run(rows)
        assert got.tolist() == plant[i0:i0 + B]
    # ties: the same maximum at several indices, across and inside slices -> the lowest index
    ties = [[5, 6], [per - 1, per], [per, 7 * per + 3, V - 1], [V - 2, V - 1], [3 * per - 1, 3 * per, 3 * per + 1], [0, V - 1]]
    rows = []
    for idxs in ties[:B]:
        r = base.clone()
        r[torch.tensor(idxs)] = 100.0
        rows.append(r)
    assert run(rows).tolist() == [min(t) for t in ties[:B]]
    # flat rows: all equal, all at the sentinel the reference uses for "minus infinity" (worker_config.h:38), all zero
    flat = [torch.full((V,), v, dtype=torch.bfloat16) for v in (1.5, -5e4, 0.0, -65504.0)]
    assert run(flat[:B]).tolist() == [0] * min(B, 4)
    # negative-only row whose maximum is the last element of the last (short) slice
    r = torch.full((V,), -3.0, dtype=torch.bfloat16)
    r[V - 1] = -2.0
    assert run([r]).tolist() == [V - 1]
    assert mpk.stats()["aborted"] == 0
    mpk.finalize()


def _zero_q(lw):
    lw["q_proj"].zero_()


@pytest.mark.parametrize("L_cached,n_new,width", [(0, 1, "small"), (0, 1, "full"), (300, 1, "small"), (517, 1, "full"), (100, 16, "full"), (0, 16, "full")])
def test_attention_closed_forms(L_cached, n_new, width):
    """q = 0 makes every score equal, so the attention output is the mean of the V rows a token sees (cached rows, and
    the rows of its own chunk up to itself): exactly representable weights 1/L, no dependence on K.  With one position
    the output is that position's V row bit for bit.  16 tokens at full width run the matrix-core form."""
    from oracle.qwen3_ref import Qwen3Config
    from test_qwen3_layer import _run_layer
    cfg = Qwen3Config(num_layers=1) if width == "full" else Qwen3Config(hidden_size=1024, num_q_heads=8, num_kv_heads=2, head_dim=128,
                                                                         intermediate_size=1536, num_layers=1)
    res = _run_layer(cfg, L_cached, n_new, "fleet", seed=77 + L_cached + n_new, mutate=_zero_q)
    nq, nkv, D = cfg.num_q_heads, cfg.num_kv_heads, cfg.head_dim
    qpk = nq // nkv
    assert bool((res["qws_gpu"] == 0).all()), "q rows must be zero"
    v_new = res["qkv_gpu"].view(n_new, nkv, qpk + 2, D)[:, :, qpk + 1]          # [T, nkv, D] as the QKV stage produced them
    v_all = torch.cat([res["cache"].v[0, :L_cached], v_new], 0).float()         # [L_cached + T, nkv, D]
    attn = res["attn_gpu"].view(n_new, nkv, qpk, D)
    for t in range(n_new):
        L = L_cached + t + 1
        want = v_all[:L].mean(0)                                                # [nkv, D]
        for j in range(qpk):
            if L == 1:
                assert torch.equal(attn[t, :, j], v_new[t]), "one position: the output must be its V row exactly"
            else:
                ulp, mabs = bf16_ulp_diff(attn[t, :, j], want.to(torch.bfloat16), floor=1.0 / 16)
                assert ulp <= 1.0, f"token {t} q head {j}: mean of {L} V rows off by {ulp} ulp ({mabs})"
    assert res["stats"]["aborted"] == 0
