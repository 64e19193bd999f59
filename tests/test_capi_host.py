"""CPU-only checks of the drop-in boundary: the shared library loads and exports every symbol include/fleet_mk.h declares,
and the host side (graph recording, validation, lowering to the stage program, reference-schema task graph) behaves as
the reference's host code does for this path -- without launching anything (host-only graphs, device = -1)."""
import ctypes
import json
import os
import re

import pytest
import torch

import mirage as mi
from mirage import _capi
from helpers import make_meta

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "fleet_mk.h")).read()
    declared = sorted(set(re.findall(r"\b(mk_[a-z_0-9]+)\s*\(", header)))
    assert len(declared) >= 20
    lib = _capi.load()
    for sym in declared:
        assert hasattr(lib, sym), f"libfleet_mk.so does not export {sym}"
    assert set(declared) == set(_capi.EXPORTED_SYMBOLS)
    assert b"gfx950" in lib.mk_version()


def test_status_codes_and_error_strings():
    lib = _capi.load()
    assert lib.mk_graph_create(None, None) == _capi.MK_EINVAL
    assert b"null" in lib.mk_last_error()
    cfg = _capi.MkConfig()
    cfg.device = -1
    cfg.max_num_batched_tokens = 65  # above the kernel's limit
    cfg.max_num_batched_requests, cfg.page_size, cfg.max_num_pages, cfg.max_seq_length = 1, 16, 4, 32
    h = ctypes.c_void_p()
    assert lib.mk_graph_create(ctypes.byref(cfg), ctypes.byref(h)) == _capi.MK_EINVAL
    assert b"max_num_batched_tokens" in lib.mk_last_error()
    cfg.max_num_batched_tokens = 1
    cfg.max_num_pages, cfg.page_size, cfg.max_seq_length = 1, 16, 64  # one sequence does not fit in the page pool
    assert lib.mk_graph_create(ctypes.byref(cfg), ctypes.byref(h)) == _capi.MK_EINVAL


def _host_mpk(B=4, R=2, max_seq=64, pages=8, page_size=16, total=2):
    meta = make_meta(total, max_seq, B, R, pages, device="cpu")
    return mi.PersistentKernel(mode="offline", world_size=1, mpi_rank=0, num_workers=256, num_local_schedulers=0, num_remote_schedulers=0,
                               max_seq_length=max_seq, max_num_batched_requests=R, max_num_batched_tokens=B, max_num_pages=pages,
                               page_size=page_size, meta_tensors=meta, profiler_tensor=None, trace_name=None, spec_decode_config=None,
                               use_cutlass_kernel=False, eos_token_id=2)


def _t(mpk, name, *shape, dtype=torch.bfloat16):
    return mpk.attach_input(torch.zeros(*shape, dtype=dtype), name)


def test_constructor_contract():
    meta = make_meta(2, 64, 4, 2, 8, device="cpu")
    kw = dict(world_size=1, mpi_rank=0, num_workers=256, num_local_schedulers=0, num_remote_schedulers=0, max_seq_length=64,
              max_num_batched_requests=2, max_num_batched_tokens=4, max_num_pages=8, page_size=16, meta_tensors=meta, profiler_tensor=None,
              trace_name=None, spec_decode_config=None, use_cutlass_kernel=False)
    with pytest.raises(ValueError, match="Invalid persistent kernel mode"):
        mi.PersistentKernel(mode="bogus", **kw)
    with pytest.raises(NotImplementedError):
        mi.PersistentKernel(mode="offline", **{**kw, "world_size": 2})
    bad = dict(meta)
    bad["tokens"] = meta["tokens"].to(torch.int32)
    with pytest.raises(AssertionError, match="tokens.dtype"):
        mi.PersistentKernel(mode="offline", **{**kw, "meta_tensors": bad})
    mpk = mi.PersistentKernel(mode="offline", **kw)
    assert mpk.total_num_requests == 2 and mpk.target_cc == 94 and mpk.max_num_batched_tokens == 4
    assert mi.mpk.spec_decode_class(None, ngram_size=3, spec_length=4) is None
    # prompt lookup is the one speculative method with tasks behind it (persistent_kernel.py:410-415); it needs the offline
    # scheduler and room for the guesses in an iteration
    pl = mi.mpk.spec_decode_class("promptlookup", ngram_size=3, spec_length=3)
    with pytest.raises(NotImplementedError, match="lookahead"):
        mi.PersistentKernel(mode="offline", **{**kw, "spec_decode_config": mi.mpk.spec_decode_class("lookahead", 3, 3)})
    with pytest.raises(NotImplementedError, match="offline"):
        mi.PersistentKernel(mode="online_notoken", **{**kw, "spec_decode_config": pl})
    with pytest.raises(ValueError, match="max_num_batched_tokens"):
        mi.PersistentKernel(mode="offline", **{**kw, "spec_decode_config": mi.mpk.spec_decode_class("promptlookup", 3, 5)})
    sp = mi.PersistentKernel(mode="offline", **{**kw, "spec_decode_config": pl})
    assert sp.spec_decode_config is pl


def test_tensor_api_and_shape_errors():
    mpk = _host_mpk()
    x = _t(mpk, "x", 4, 1024)
    assert x.num_dims == 2 and x.dim(0) == 4 and x.dim(1) == 1024
    with pytest.raises(AssertionError):  # row-major only (persistent_kernel.py:473-474)
        mpk.attach_input(torch.zeros(8, 4, dtype=torch.bfloat16).t(), "xt")
    with pytest.raises(RuntimeError, match="Invalid io_category"):
        mpk.new_tensor((4, 8), name="bad", io_category="host_tensor")
    q, k, v = _t(mpk, "q", 1024, 1024), _t(mpk, "k", 256, 1024), _t(mpk, "v", 256, 1024)
    qkv = mpk.shuffle_tensors([q, k, v], 0, 2, "qkv")
    assert qkv.dim(0) == 1536 and qkv.dim(1) == 1024
    with pytest.raises(_capi.MkError, match="not divisible"):
        mpk.shuffle_tensors([q, k, v], 0, 3, "qkv3")
    with pytest.raises(AssertionError):
        mpk.shuffle_tensors([q, k], 1, 2, "dim1")
    # unknown task names are rejected when registered, like Graph::register_task (src/kernel/graph.cc:844-847)
    with pytest.raises(_capi.MkError, match="Unsupported task name"):
        mpk._task("definitely_not_a_task", (1, 1, 1), (128, 1, 1), [(x, (-1, -1, -1), -1)])
    with pytest.raises(NotImplementedError):
        mpk.allreduce_layer()


def test_lowering_fuses_norm_and_swiglu_and_attention():
    mpk = _host_mpk(B=4, R=2)
    H, I, nq, nkv, D = 1024, 1536, 8, 2, 128
    ids = _t(mpk, "ids", 4, 1, dtype=torch.int64)
    emb, x = _t(mpk, "emb", 100, H), mpk.new_tensor((4, H), name="x")
    nw, n = _t(mpk, "nw", H), mpk.new_tensor((4, H), name="n")
    q, k, v = _t(mpk, "q", nq * D, H), _t(mpk, "k", nkv * D, H), _t(mpk, "v", nkv * D, H)
    qkv_w = mpk.shuffle_tensors([q, k, v], 0, nkv, "qkv_w")
    qkv = mpk.new_tensor((4, (nq + 2 * nkv) * D), name="qkv")
    kc, vc = _t(mpk, "kc", 8, 16, nkv, D), _t(mpk, "vc", 8, 16, nkv, D)
    qn, kn = _t(mpk, "qn", D), _t(mpk, "kn", D)
    cos, sin = _t(mpk, "cos", 64, D), _t(mpk, "sin", 64, D)
    qws, att, lse = mpk.new_tensor((4, nq * D), name="qws"), mpk.new_tensor((4, nq * D), name="att"), mpk.new_tensor((4, nq), dtype=mi.float32, name="lse")
    wo, x1 = _t(mpk, "wo", H, nq * D), mpk.new_tensor((4, H), name="x1")
    wg, wu = _t(mpk, "wg", I, H), _t(mpk, "wu", I, H)
    gu = mpk.shuffle_tensors([wg, wu], 0, I // 128, "gu")
    mid, act = mpk.new_tensor((4, 2 * I), name="mid"), mpk.new_tensor((4, I), name="act")
    wd, x2 = _t(mpk, "wd", H, I), mpk.new_tensor((4, H), name="x2")
    lm, logits = _t(mpk, "lm", 1000, H), mpk.new_tensor((4, 1000), name="logits")
    pv, pi = mpk.new_tensor((4, 8), name="pv"), mpk.new_tensor((4, 8), dtype=mi.int64, name="pi")
    out = _t(mpk, "out", 4, 1, dtype=torch.int64)
    mpk.embed_layer(input=ids, weight=emb, output=x, grid_dim=(1, 1, 1), block_dim=(128, 1, 1), input_source=1)
    mpk.rmsnorm_layer(input=x, weight=nw, output=n, grid_dim=(4, 1, 1), block_dim=(128, 1, 1))
    mpk.linear_layer(input=n, weight=qkv_w, output=qkv, grid_dim=(24, 1, 1), block_dim=(128, 1, 1))
    mpk.kv_cache_update_layer(input=qkv, k_cache=kc, v_cache=vc, q_norm=qn, k_norm=kn, cos_pos_embed=cos, sin_pos_embed=sin, q_workspace=qws,
                              grid_dim=(2, nkv, 1), block_dim=(256, 1, 1))
    mpk.paged_attention_ck_fmha_layer(q_workspace=qws, k_cache=kc, v_cache=vc, o_acc=att, lse_acc=lse, attention_params=(nq, 1, 2),
                                      grid_dim=(2, nkv, 1), block_dim=(256, 1, 1))
    mpk.linear_with_residual_layer(input=att, weight=wo, residual=x, output=x1, grid_dim=(16, 1, 1), block_dim=(256, 1, 1))
    mpk.rmsnorm_layer(input=x1, weight=nw, output=n, grid_dim=(4, 1, 1), block_dim=(128, 1, 1))
    mpk.linear_layer(input=n, weight=gu, output=mid, grid_dim=(48, 1, 1), block_dim=(128, 1, 1))
    mpk.silu_mul_layer(input=mid, output=act, grid_dim=(I // 128, 1, 1), block_dim=(128, 1, 1))
    mpk.linear_with_residual_layer(input=act, weight=wd, residual=x1, output=x2, grid_dim=(16, 1, 1), block_dim=(256, 1, 1))
    mpk.rmsnorm_layer(input=x2, weight=nw, output=n, grid_dim=(4, 1, 1), block_dim=(128, 1, 1))
    mpk.linear_layer(input=n, weight=lm, output=logits, grid_dim=(8, 1, 1), block_dim=(128, 1, 1))
    mpk.argmax_partial_layer(input=logits, output=(pv, pi), grid_dim=(8, 1, 1), block_dim=(128, 1, 1))
    mpk.argmax_reduce_layer(input=(pv, pi), output=out, grid_dim=(1, 1, 1), block_dim=(128, 1, 1))
    prog = [l.split(None, 1)[1] for l in mpk.describe_program().splitlines()]
    kinds = [l.split()[0] for l in prog]
    assert kinds == ["EMBED", "NORM[multi-token", "LINEAR+norm", "ATTN", "LINEAR+res", "NORM[multi-token", "LINEAR+norm+silu", "LINEAR+res",
                     "NORM[multi-token", "LINEAR+norm", "ARGMAX_PARTIAL", "ARGMAX_REDUCE"]
    assert "segs=3" in prog[2] and "segs=2" in prog[6] and "-> act" in prog[6]  # shuffled views resolved, activation folded in
    # reference-shaped task graph: tasks = 2 + sum of grid sizes; first/last events as in runtime.cc:176-182,590-595
    tg = json.loads(mpk.kn_graph.generate_task_graph(1, 0)["json_file"])
    n_tasks = 2 + 1 + 4 + 24 + 4 + 4 + 16 + 4 + 48 + 12 + 16 + 4 + 8 + 8 + 1
    assert len(tg["all_tasks"]) == n_tasks
    assert tg["all_tasks"][0]["task_type"] == 0 and tg["all_tasks"][1]["task_type"] == 10
    assert tg["all_events"][0]["event_type"] == 911 and tg["all_events"][1]["event_type"] == 903 and tg["all_events"][-1]["event_type"] == 910
    assert tg["all_events"][1]["first_task_id"] == 2 and tg["all_events"][1]["last_task_id"] == n_tasks
    lin = [t for t in tg["all_tasks"] if t["task_type"] == 120]
    # 1536 rows over 24 blocks; a shuffled weight is named by the source its slice starts in (runtime.cc:1229-1283):
    # groups of [q 512 ; k 128 ; v 128] -> block 1 = q rows 64.., block 9 = k rows 64.., block 13 = q rows 576..
    w1, w9, w13 = lin[1]["inputs"][1], lin[9]["inputs"][1], lin[13]["inputs"][1]
    assert (w1["base_ptr"], w1["offset"], w1["dims"], w1["strides"]) == ("q", 64 * 1024 * 2, [64, 1024], [1024, 1])
    assert (w9["base_ptr"], w9["offset"]) == ("k", 64 * 1024 * 2) and (w13["base_ptr"], w13["offset"]) == ("q", 576 * 1024 * 2)
    assert lin[1]["outputs"][0]["offset"] == 64 * 2
    assert tg["first_tasks"] == [2] and tg["all_tasks"][2]["dependent_event"] == 0x7FFFFFFFFFFFFFFE
    for key in ("trigger_event", "dependent_event", "request_id", "expert_offset", "kv_idx", "merge_task_offset", "n_tile_start", "n_tile_count"):
        assert key in lin[0]
    with pytest.raises(_capi.MkError, match="one GPU"):
        mpk.kn_graph.generate_task_graph(2, 1)
    with pytest.raises(_capi.MkError, match="without a device"):
        mpk.compile()


def _events(tg):
    return [(e["event_type"], e["num_triggers"], e["first_task_id"], e["last_task_id"]) for e in tg["all_events"]]


def test_task_graph_events_follow_the_reference_partition_rule():
    """Events between two operators as src/kernel/runtime.cc:53-140,519-612 builds them, expected values derived by hand:
    one tensor carries the dependency; along each of its dims there are gcd(producer partition, consumer partition)
    events; an event owns the consumer blocks of its slice (stored event by event, in bid order inside an event) and counts
    the producer blocks of the matching slice."""
    INV, EMPTY = 0x7FFFFFFFFFFFFFFE, 900
    # (i) norm (4) -> 96-block QKV linear -> kv_cache_update (2, 8, 1) -> attention (2, 8, 1) -> o projection (16)
    mpk = _host_mpk(B=4, R=2)
    H, nq, nkv, D = 1024, 32, 8, 128
    x, nw, n = mpk.new_tensor((4, H), name="x"), _t(mpk, "nw", H), mpk.new_tensor((4, H), name="n")
    qkv_w = mpk.shuffle_tensors([_t(mpk, "q", nq * D, H), _t(mpk, "k", nkv * D, H), _t(mpk, "v", nkv * D, H)], 0, nkv, "qkv_w")
    qkv = mpk.new_tensor((4, (nq + 2 * nkv) * D), name="qkv")
    kc, vc = _t(mpk, "kc", 8, 16, nkv, D), _t(mpk, "vc", 8, 16, nkv, D)
    qws, att, lse = mpk.new_tensor((4, nq * D), name="qws"), mpk.new_tensor((4, nq * D), name="att"), mpk.new_tensor((4, nq), dtype=mi.float32, name="lse")
    mpk.rmsnorm_layer(input=x, weight=nw, output=n, grid_dim=(4, 1, 1), block_dim=(128, 1, 1))
    mpk.linear_layer(input=n, weight=qkv_w, output=qkv, grid_dim=(96, 1, 1), block_dim=(128, 1, 1))
    mpk.kv_cache_update_layer(input=qkv, k_cache=kc, v_cache=vc, q_norm=_t(mpk, "qn", D), k_norm=_t(mpk, "kn", D), cos_pos_embed=_t(mpk, "cos", 64, D),
                              sin_pos_embed=_t(mpk, "sin", 64, D), q_workspace=qws, grid_dim=(2, nkv, 1), block_dim=(256, 1, 1))
    mpk.paged_attention_ck_fmha_layer(q_workspace=qws, k_cache=kc, v_cache=vc, o_acc=att, lse_acc=lse, attention_params=(nq, 1, 2),
                                      grid_dim=(2, nkv, 1), block_dim=(256, 1, 1))
    mpk.linear_with_residual_layer(input=att, weight=_t(mpk, "wo", H, nq * D), residual=x, output=mpk.new_tensor((4, H), name="x1"),
                                   grid_dim=(16, 1, 1), block_dim=(256, 1, 1))
    tg = json.loads(mpk.kn_graph.generate_task_graph(1, 0)["json_file"])
    n_tasks = 2 + 4 + 96 + 16 + 16 + 16
    expect = [(911, 1, 0, 0), (903, 1, 2, n_tasks),
              (EMPTY, 4, 6, 102)]                                       # the 4 norm rows -> all 96 linear blocks (the linear reads whole rows)
    expect += [(EMPTY, 12, 102 + 2 * i, 104 + 2 * i) for i in range(8)]  # gcd(96, 8) = 8 slices of the qkv columns: 12 blocks -> kv head i of both requests
    expect += [(EMPTY, 16, 118, 134), (EMPTY, 16, 134, 150), (910, 16, 0, 0)]
    assert _events(tg) == expect
    T = tg["all_tasks"]
    assert tg["first_tasks"] == [2, 3, 4, 5]
    assert [t["trigger_event"] for t in T[2:6]] == [2] * 4 and [t["dependent_event"] for t in T[2:6]] == [INV] * 4
    assert [t["trigger_event"] for t in T[6:102]] == [3 + b // 12 for b in range(96)] and all(t["dependent_event"] == 2 for t in T[6:102])
    # kv_cache_update tasks are stored event by event: (request 0, head i), (request 1, head i)
    assert [(t["request_id"], t["dependent_event"]) for t in T[102:118]] == [(r, 3 + h) for h in range(8) for r in range(2)]
    assert [t["inputs"][0]["offset"] for t in T[102:118]] == [h * 768 * 2 for h in range(8) for r in range(2)]
    assert all(t["trigger_event"] == 11 for t in T[102:118]) and all(t["trigger_event"] == 12 for t in T[118:134])
    assert [t["request_id"] for t in T[118:134]] == [r for r in range(2) for h in range(8)]  # plain bid order again
    assert [(t["kv_idx"], t["merge_task_offset"]) for t in T[118:134]] == [(0, h) for r in range(2) for h in range(8)]
    assert all(t["trigger_event"] == 13 and t["dependent_event"] == 12 for t in T[134:150])
    # a task type that sets no metadata still carries request_id = bid.x in a union that started as all ones
    assert (T[7]["request_id"], T[7]["n_tile_start"], T[7]["kv_idx"], T[7]["n_tile_count"], T[7]["merge_task_offset"], T[7]["expert_offset"]) == (1, 1, 65535, 65535, -1, -65535)
    assert T[6]["variant_id"] == 0 and T[134]["variant_id"] == 0 and T[0]["trigger_event"] == INV and T[1]["trigger_event"] == 1

    # (ii) two grids partitioned along both dims of the shared [8, 512] tensor: producer (8 column blocks, 4 row blocks),
    # consumer (6, 2): rows gcd(4, 2) = 2 slices, columns gcd(8, 1) = 1
    mpk = _host_mpk(B=8, R=2, pages=8)
    a, y, z = mpk.new_tensor((8, 1024), name="a"), mpk.new_tensor((8, 512), name="y"), mpk.new_tensor((8, 384), name="z")
    mpk.linear_m_parallel_layer(input=a, weight=_t(mpk, "W1", 512, 1024), output=y, grid_dim=(8, 4, 1), block_dim=(128, 1, 1))
    mpk.linear_with_residual_m_parallel_layer(input=y, weight=_t(mpk, "W2", 384, 512), residual=mpk.new_tensor((8, 384), name="r"), output=z,
                                              grid_dim=(6, 2, 1), block_dim=(128, 1, 1))
    tg = json.loads(mpk.kn_graph.generate_task_graph(1, 0)["json_file"])
    assert _events(tg) == [(911, 1, 0, 0), (903, 1, 2, 46), (EMPTY, 16, 34, 40), (EMPTY, 16, 40, 46), (910, 12, 0, 0)]
    T = tg["all_tasks"]
    assert [t["trigger_event"] for t in T[2:34]] == [2 + (i % 4) // 2 for i in range(32)]  # task 2 + 4 x + y waits on the slice of row block y
    assert [(t["request_id"], t["inputs"][0]["offset"]) for t in T[34:46]] == [(xb, yb * 4 * 512 * 2) for yb in range(2) for xb in range(6)]
    assert [t["dependent_event"] for t in T[34:46]] == [2] * 6 + [3] * 6 and all(t["trigger_event"] == 4 for t in T[34:46])

    # (iii) mixture of experts: W13 (10, 24) -> activation (tokens 4, slots 8) -> W2 (8, 32) -> weighted sum (4, 8)
    mpk = _host_mpk(B=4, R=2)
    E, topk, Hm, Im = 16, 8, 2048, 768
    xin, lg = mpk.new_tensor((4, Hm), name="xin"), mpk.new_tensor((4, E), name="lg")
    tw, ri, mk = mpk.new_tensor((4, topk), dtype=mi.float32, name="tw"), mpk.new_tensor((E, 4), dtype=mi.int32, name="ri"), mpk.new_tensor((E + 1,), dtype=mi.int32, name="mk")
    mid, act, eo = mpk.new_tensor((4, topk, 2 * Im), name="mid"), mpk.new_tensor((4, topk, Im), name="act"), mpk.new_tensor((4, topk, Hm), name="eo")
    res, out = mpk.new_tensor((4, Hm), name="res"), mpk.new_tensor((4, Hm), name="out")
    mpk.moe_topk_softmax_routing_layer(input=lg, output=(tw, ri, mk), grid_dim=(1, 1, 1), block_dim=(256, 1, 1))
    mpk.moe_w13_linear_layer(input=xin, weight=_t(mpk, "w13", E, 2 * Im, Hm), moe_routing_indices=ri, moe_mask=mk, output=mid, grid_dim=(10, 24, 1), block_dim=(256, 1, 1))
    mpk.moe_silu_mul_layer(input=mid, output=act, grid_dim=(4, topk, 1), block_dim=(256, 1, 1))
    mpk.moe_w2_linear_layer(input=act, weight=_t(mpk, "w2", E, Hm, Im), moe_routing_indices=ri, moe_mask=mk, output=eo, grid_dim=(8, 32, 1), block_dim=(256, 1, 1))
    mpk.moe_mul_sum_add_layer(input=eo, weight=tw, residual=res, output=out, grid_dim=(4, 8, 1), block_dim=(256, 1, 1))
    tg = json.loads(mpk.kn_graph.generate_task_graph(1, 0)["json_file"])
    base_w2, base_sum = 2 + 1 + 240 + 32, 2 + 1 + 240 + 32 + 256
    expect = [(911, 1, 0, 0), (903, 1, 2, base_sum + 32), (EMPTY, 1, 3, 243), (EMPTY, 240, 243, 275), (EMPTY, 32, base_w2, base_sum)]
    # the expert outputs [4, 8, 2048] are cut in 32 column blocks by W2 and in 8 by the weighted sum: gcd = 8 events, each
    # fired by 8 x 4 W2 blocks and owning the four tokens' tasks of column block i
    expect += [(EMPTY, 32, base_sum + 4 * i, base_sum + 4 * i + 4) for i in range(8)] + [(910, 32, 0, 0)]
    assert _events(tg) == expect
    T = tg["all_tasks"]
    assert [t["expert_offset"] for t in T[3:243]] == [(yb << 16) | xb for xb in range(10) for yb in range(24)]  # moe tasks pack (bid.y, bid.x)
    assert [t["trigger_event"] for t in T[base_w2:base_sum]] == [5 + yb // 4 for xb in range(8) for yb in range(32)]
    assert [(t["request_id"], t["dependent_event"]) for t in T[base_sum:base_sum + 32]] == [(tok, 5 + i) for i in range(8) for tok in range(4)]
    assert [t["outputs"][0]["offset"] for t in T[base_sum:base_sum + 32]] == [(tok * Hm + i * 256) * 2 for i in range(8) for tok in range(4)]

    # gang tasks: one task per die; n_tile_count = tiles per die, attention tasks also their first work item
    mpk = _host_mpk(B=4, R=2)
    n2, w8 = mpk.new_tensor((4, H), name="n"), _t(mpk, "w8", 4096, H)
    o8 = mpk.new_tensor((4, 4096), name="o8")
    mpk.gang_rmsnorm_layer(input=mpk.new_tensor((4, H), name="x"), weight=_t(mpk, "nw", H), output=n2)
    mpk.gang_linear_layer(input=n2, weight=w8, output=o8, tile_n=64, output_stride=4096, m_tiles=1)
    tg = json.loads(mpk.kn_graph.generate_task_graph(1, 0)["json_file"])
    T = tg["all_tasks"]
    assert _events(tg) == [(911, 1, 0, 0), (903, 1, 2, 18), (EMPTY, 8, 10, 18), (910, 8, 0, 0)]
    assert [(t["n_tile_start"], t["n_tile_count"]) for t in T[2:10]] == [(0, 4)] * 8       # gang_rmsnorm: params[0] = batch rows
    assert [(t["n_tile_start"], t["n_tile_count"]) for t in T[10:18]] == [(0, 8)] * 8      # 4096 / 8 dies / 64 = 8 tiles per die
    assert [t["inputs"][1]["offset"] for t in T[10:18]] == [d * 512 * H * 2 for d in range(8)]  # die d streams weight chunk d


def test_lowering_rejects_bad_graphs():
    mpk = _host_mpk()
    x, W = _t(mpk, "x", 4, 1024), _t(mpk, "W", 512, 1000)
    y = mpk.new_tensor((4, 512), name="y")
    mpk.linear_layer(input=x, weight=W, output=y, grid_dim=(8, 1, 1), block_dim=(128, 1, 1))
    with pytest.raises(_capi.MkError, match="expected 1024"):
        mpk.describe_program()
    mpk2 = _host_mpk()
    x, W = _t(mpk2, "x", 2, 1024), _t(mpk2, "W", 512, 1024)  # fewer rows than max_num_batched_tokens
    y = mpk2.new_tensor((4, 512), name="y")
    mpk2.linear_layer(input=x, weight=W, output=y, grid_dim=(8, 1, 1), block_dim=(128, 1, 1))
    with pytest.raises(_capi.MkError, match="max_num_batched_tokens"):
        mpk2.describe_program()
    mpk3 = _host_mpk()
    qkv = _t(mpk3, "qkv", 4, 12 * 64)
    kc, vc = _t(mpk3, "kc", 8, 16, 2, 64), _t(mpk3, "vc", 8, 16, 2, 64)
    o, lse, qws = mpk3.new_tensor((4, 512), name="o"), mpk3.new_tensor((4, 8), dtype=mi.float32, name="lse"), mpk3.new_tensor((4, 512), name="qws")
    mpk3.gang_paged_attention_split_kv_layer(input=qkv, k_cache=kc, v_cache=vc, q_norm=None, k_norm=None, cos_pos_embed=None, sin_pos_embed=None,
                                             lse=lse, output=o, q_workspace=qws, attention_params=(8, 1, 512))
    with pytest.raises(_capi.MkError, match="head_dim 64"):
        mpk3.describe_program()
    mpk4 = _host_mpk()
    with pytest.raises(AssertionError, match="divisible"):  # gang layers need N divisible by 8 * tile_n (persistent_kernel.py:1595-1599)
        mpk4.gang_linear_layer(input=_t(mpk4, "x", 4, 1024), weight=_t(mpk4, "W", 1000, 1024), output=mpk4.new_tensor((4, 1000), name="y"),
                               tile_n=64, output_stride=1000)


def _moe_graph(mpk, B, gang, fused_order=True):
    H, E, topk, MI = 512, 16, 4, 128
    x, n = mpk.new_tensor((B, H), name="x"), mpk.new_tensor((B, H), name="n")
    nw, wr = _t(mpk, "nw", H), _t(mpk, "router", E, H)
    w13, w2 = _t(mpk, "w13", E, 2 * MI, H), _t(mpk, "w2", E, H, MI)
    gate = mpk.new_tensor((B, E), name="gate")
    tw = mpk.new_tensor((B, topk), dtype=mi.float32, name="topk_w")
    ri = mpk.new_tensor((E, B), dtype=mi.int32, name="routing")
    mask = mpk.new_tensor((E + 1,), dtype=mi.int32, name="mask")
    mid, act, y = mpk.new_tensor((B, topk, 2 * MI), name="mid"), mpk.new_tensor((B, topk, MI), name="act"), mpk.new_tensor((B, topk, H), name="y")
    out = mpk.new_tensor((B, H), name="out")
    mpk.rmsnorm_layer(input=x, weight=nw, output=n, grid_dim=(B, 1, 1), block_dim=(128, 1, 1))
    mpk.linear_layer(input=n, weight=wr, output=gate, grid_dim=(1, 1, 1), block_dim=(256, 1, 1))
    mpk.moe_topk_softmax_routing_layer(input=gate, output=(tw, ri, mask), grid_dim=(1, 1, 1), block_dim=(256, 1, 1))
    if gang:
        mpk.gang_moe_w13_linear_layer(input=n, weight=w13, moe_routing_indices=ri, moe_mask=mask, output=mid)
    else:
        mpk.moe_w13_linear_layer(input=n, weight=w13, moe_routing_indices=ri, moe_mask=mask, output=mid, grid_dim=(10, 2 * MI // 64, 1), block_dim=(256, 1, 1))
    mpk.moe_silu_mul_layer(input=mid, output=act, grid_dim=(B, topk, 1), block_dim=(256, 1, 1))
    if gang:
        mpk.gang_moe_w2_linear_layer(input=act, weight=w2, moe_routing_indices=ri, moe_mask=mask, output=y)
    else:
        mpk.moe_w2_linear_layer(input=act, weight=w2, moe_routing_indices=ri, moe_mask=mask, output=y, grid_dim=(8, H // 64, 1), block_dim=(256, 1, 1))
    mpk.moe_mul_sum_add_layer(input=y, weight=tw, residual=x, output=out, grid_dim=(B, H // 256, 1), block_dim=(256, 1, 1))
    return dict(E=E, topk=topk, MI=MI, H=H)


@pytest.mark.parametrize("gang", [False, True])
def test_lowering_of_mixture_of_experts_layers(gang):
    """The reference's MoE sequence (demo/qwen3/demo_30B_A3B.py:675-754) lowers to router linear, top-k stage (multi-token only),
    W13 with routing + SwiGLU folded in, W2 with the combine folded in for single tokens, and a multi-token combine stage."""
    mpk = _host_mpk(B=4, R=2)
    d = _moe_graph(mpk, 4, gang)
    prog = [l.split(None, 1)[1] for l in mpk.describe_program().splitlines()]
    kinds = [l.split()[0] for l in prog]
    assert kinds == ["NORM[multi-token", "LINEAR+norm", "MOE_TOPK[multi-token", "MOE_LINEAR+route(single", "MOE_LINEAR", "MOE_COMBINE[multi-token"]
    assert "+silu -> act" in prog[3] and "n=256 k=512" in prog[3] and "+combine(single token) -> out" in prog[4] and "n=512 k=128" in prog[4]
    tg = json.loads(mpk.kn_graph.generate_task_graph(1, 0)["json_file"])
    types = {t["task_type"] for t in tg["all_tasks"]}
    # runtime_header.h:141-146 task ids
    assert ({174, 175} if gang else {170, 171}) <= types and {172, 173, 118} <= types


def test_lowering_rejects_bad_moe_graphs():
    mpk = _host_mpk(B=2, R=2)
    H, E, topk = 256, 8, 2
    gate = mpk.new_tensor((2, E), name="gate")
    tw = mpk.new_tensor((2, topk), dtype=mi.float32, name="tw")
    ri = mpk.new_tensor((E, 2), dtype=mi.int32, name="ri")
    mask = mpk.new_tensor((E + 1,), dtype=mi.int32, name="mask")
    mpk.moe_topk_softmax_routing_layer(input=gate, output=(tw, ri, mask), grid_dim=(1, 1, 1), block_dim=(256, 1, 1))
    with pytest.raises(_capi.MkError, match="must be followed by the per-expert linear"):
        mpk.describe_program()
    mpk = _host_mpk(B=2, R=2)
    n, w = mpk.new_tensor((2, H), name="n"), _t(mpk, "w", E, 64, H + 8)
    ri = mpk.new_tensor((E, 2), dtype=mi.int32, name="ri")
    mask = mpk.new_tensor((E + 1,), dtype=mi.int32, name="mask")
    y = mpk.new_tensor((2, topk, 64), name="y")
    mpk.moe_w13_linear_layer(input=n, weight=w, moe_routing_indices=ri, moe_mask=mask, output=y, grid_dim=(1, 1, 1), block_dim=(256, 1, 1))
    with pytest.raises(_capi.MkError, match=r"input must be \[tokens, 264\]"):
        mpk.describe_program()


def _attn_tensors(mpk, nq=8, nkv=2, D=128, chunks=1, pages=8):
    t = dict(qkv=_t(mpk, "qkv", 4, (nq + 2 * nkv) * D), kc=_t(mpk, "kc", pages, 16, nkv, D), vc=_t(mpk, "vc", pages, 16, nkv, D), qn=_t(mpk, "qn", D),
             kn=_t(mpk, "kn", D), cos=_t(mpk, "cos", 64, D), sin=_t(mpk, "sin", 64, D), out=mpk.new_tensor((4, nq * D), name="attn_out"),
             qws=mpk.new_tensor((4, nq * D), name="qws"))
    t["lse"] = mpk.new_tensor((4, nkv * chunks * (nq // nkv)), dtype=mi.float32, name="lse")
    t["oacc"] = mpk.new_tensor((4, nkv * chunks * (nq // nkv) * D), dtype=mi.float32, name="o_acc")
    return t


def test_every_attention_flavour_lowers_to_one_stage():
    """The reference API has five ways to say "attention" (persistent_kernel.py:724-1180); with or without a KV split in
    the graph each becomes ONE stage that writes the final bf16 output (the merge task's output when chunks > 1)."""
    nq, nkv, D = 8, 2, 128
    kw = dict(q_norm=None, k_norm=None, cos_pos_embed=None, sin_pos_embed=None)

    def program(build):
        mpk = _host_mpk(B=4, R=2)
        build(mpk)
        return [l.split(None, 1)[1] for l in mpk.describe_program().splitlines()]

    def fused(mpk):
        t = _attn_tensors(mpk)
        mpk.paged_attention_layer(input=t["qkv"], k_cache=t["kc"], v_cache=t["vc"], q_norm=t["qn"], k_norm=t["kn"], cos_pos_embed=t["cos"],
                                  sin_pos_embed=t["sin"], output=t["out"], grid_dim=(2, nkv, 1), block_dim=(128, 1, 1))
    p = program(fused)
    assert len(p) == 1 and p[0].startswith("ATTN qkv -> attn_out") and "norm=1 rope=1" in p[0]

    def split(mpk):
        t = _attn_tensors(mpk)
        lse3 = mpk.new_tensor((4, 3 * (nq // nkv), nkv), dtype=mi.float32, name="lse3")
        tmp3 = mpk.new_tensor((4, 3 * (nq // nkv) * D, nkv), name="tmp3")
        mpk.paged_attention_split_kv_layer(input=t["qkv"], k_cache=t["kc"], v_cache=t["vc"], lse=lse3, output=tmp3, attention_params=(nq, 3),
                                           grid_dim=(2, nkv, 3), block_dim=(128, 1, 1), **kw)
        mpk.paged_attention_split_kv_merge_layer(lse=lse3, output_tmp=tmp3, output=t["out"], attention_params=(nq, D), grid_dim=(2, nkv, 1),
                                                 block_dim=(128, 1, 1))
    p = program(split)
    assert len(p) == 1 and p[0].startswith("ATTN qkv -> attn_out") and "norm=0 rope=0" in p[0]

    def ck_chunks(mpk):
        t = _attn_tensors(mpk, chunks=4)
        mpk.kv_cache_update_layer(input=t["qkv"], k_cache=t["kc"], v_cache=t["vc"], q_norm=t["qn"], k_norm=t["kn"], cos_pos_embed=t["cos"],
                                  sin_pos_embed=t["sin"], q_workspace=t["qws"], grid_dim=(2, nkv, 1), block_dim=(256, 1, 1))
        mpk.paged_attention_ck_fmha_layer(q_workspace=t["qws"], k_cache=t["kc"], v_cache=t["vc"], o_acc=t["oacc"], lse_acc=t["lse"],
                                          attention_params=(nq, 4, 2), grid_dim=(2, nkv, 4), block_dim=(256, 1, 1))
        mpk.paged_attention_ck_fmha_merge_layer(lse=t["lse"], output_tmp=t["oacc"], output=t["out"], attention_params=(nq, D, 4, nkv),
                                                grid_dim=(2, nkv, 1), block_dim=(256, 1, 1))
    p = program(ck_chunks)
    assert len(p) == 1 and p[0].startswith("ATTN qkv -> attn_out")

    def gang_chunks(mpk):
        t = _attn_tensors(mpk, chunks=2)
        mpk.gang_paged_attention_split_kv_layer(input=t["qkv"], k_cache=t["kc"], v_cache=t["vc"], q_norm=t["qn"], k_norm=t["kn"],
                                                cos_pos_embed=t["cos"], sin_pos_embed=t["sin"], lse=t["lse"], output=t["oacc"],
                                                q_workspace=t["qws"], attention_params=(nq, 2, nq * D))
        mpk.gang_paged_attention_split_kv_merge_layer(lse=t["lse"], output_tmp=t["oacc"], output=t["out"], attention_params=(nq, D, nkv, 2))
    p = program(gang_chunks)
    assert len(p) == 1 and p[0].startswith("ATTN qkv -> attn_out")

    def missing_merge(mpk):
        t = _attn_tensors(mpk, chunks=2)
        mpk.gang_paged_attention_split_kv_layer(input=t["qkv"], k_cache=t["kc"], v_cache=t["vc"], q_norm=t["qn"], k_norm=t["kn"],
                                                cos_pos_embed=t["cos"], sin_pos_embed=t["sin"], lse=t["lse"], output=t["oacc"],
                                                q_workspace=t["qws"], attention_params=(nq, 2, nq * D))
    with pytest.raises(_capi.MkError, match="must be followed by gang_attn_merge_mi300"):
        program(missing_merge)

    def lone_merge(mpk):
        t = _attn_tensors(mpk, chunks=2)
        mpk.gang_paged_attention_split_kv_merge_layer(lse=t["lse"], output_tmp=t["oacc"], output=t["out"], attention_params=(nq, D, nkv, 2))
    with pytest.raises(_capi.MkError, match="must directly follow"):
        program(lone_merge)

    def small_cache(mpk):
        t = _attn_tensors(mpk, pages=4)  # the configuration has 8 pages
        mpk.gang_paged_attention_split_kv_layer(input=t["qkv"], k_cache=t["kc"], v_cache=t["vc"], q_norm=t["qn"], k_norm=t["kn"],
                                                cos_pos_embed=t["cos"], sin_pos_embed=t["sin"], lse=t["lse"], output=t["out"],
                                                q_workspace=t["qws"], attention_params=(nq, 1, nq * D))
    with pytest.raises(_capi.MkError, match="fewer than max_num_pages"):
        program(small_cache)

    def extend(mpk):  # the speculating request's rows (persistent_kernel.py:653): the cache form with one page per request
        t = _attn_tensors(mpk)
        mpk.single_batch_extend_attention_layer(input=t["qkv"], k_cache=t["kc"], v_cache=t["vc"], q_norm=t["qn"], k_norm=t["kn"],
                                                cos_pos_embed=t["cos"], sin_pos_embed=t["sin"], output=t["out"], grid_dim=(1, nkv, 1), block_dim=(128, 1, 1))
    p = program(extend)
    assert len(p) == 1 and p[0].startswith("ATTN qkv -> attn_out") and "norm=1 rope=1" in p[0]


def test_split_k_pair_and_fused_activation_lower_to_linear_stages():
    """The reference's model builder for this GPU family (mpk/models/qwen3/builder.py:395-420,560-585,700-712) writes QKV
    and o_proj as splitk_linear into an fp32 workspace + splitk_reduce, and the MLP tail as silu_mul_linear_with_residual."""
    mpk = _host_mpk(B=4, R=2)
    H, I = 1024, 1536
    x, n, nw = mpk.new_tensor((4, H), name="x"), mpk.new_tensor((4, H), name="n"), _t(mpk, "nw", H)
    W, ws = _t(mpk, "W", H, H), mpk.attach_input(torch.zeros(4 * 4, H, dtype=torch.float32), "splitk_ws")
    y = mpk.new_tensor((4, H), name="y")
    mpk.rmsnorm_layer(input=x, weight=nw, output=n, grid_dim=(4, 1, 1), block_dim=(128, 1, 1))
    mpk.splitk_linear_layer(input=n, weight=W, output=ws, grid_dim=(H // 128, 4, 1), block_dim=(256, 1, 1))
    mpk.splitk_reduce_layer(workspace=ws, residual=x, output=y, k_splits=4, grid_dim=(H // 128, 1, 1), block_dim=(256, 1, 1))
    wg, wu = _t(mpk, "wg", I, H), _t(mpk, "wu", I, H)
    gu = mpk.shuffle_tensors([wg, wu], 0, 6, "gu")  # groups of [gate256 ; up256]
    mid = mpk.attach_input(torch.zeros(4, 2 * I, dtype=torch.bfloat16), "mlp_mid")
    wd, out = _t(mpk, "wd", H, I), mpk.new_tensor((4, H), name="out")
    mpk.rmsnorm_layer(input=y, weight=nw, output=n, grid_dim=(4, 1, 1), block_dim=(128, 1, 1))
    mpk.linear_layer(input=n, weight=gu, output=mid, grid_dim=(12, 1, 1), block_dim=(128, 1, 1))
    mpk.silu_mul_linear_with_residual_layer(input=mid, weight=wd, residual=y, output=out, grid_dim=(H // 64, 1, 1), block_dim=(256, 1, 1))
    prog = [l.split(None, 1)[1] for l in mpk.describe_program().splitlines()]
    kinds = [l.split()[0] for l in prog]
    assert kinds == ["NORM[multi-token", "LINEAR+norm+res", "NORM[multi-token", "LINEAR+norm", "LINEAR+res"]
    assert "-> y" in prog[1] and "+silu half=256 " in prog[3] and "folded in" in prog[3] and "silu_mul(mlp_mid) x wd -> out" in prog[4] and "k=1536" in prog[4]
    # a physical gate/up weight: [gate | up] halves as the reference task kernel reads them (whatever the producer's grid),
    # unless the caller that interleaved it says how
    for kw, half in (({}, I), ({"gate_rows_per_group": 128}, 128)):
        mpk = _host_mpk(B=4, R=2)
        n, guw = mpk.new_tensor((4, H), name="n"), _t(mpk, "gu", 2 * I, H)
        mid, wd, y, out = mpk.new_tensor((4, 2 * I), name="mid"), _t(mpk, "wd", H, I), mpk.new_tensor((4, H), name="y"), mpk.new_tensor((4, H), name="out")
        mpk.linear_layer(input=n, weight=guw, output=mid, grid_dim=(24, 1, 1), block_dim=(128, 1, 1))
        mpk.silu_mul_linear_with_residual_layer(input=mid, weight=wd, residual=y, output=out, grid_dim=(H // 64, 1, 1), block_dim=(256, 1, 1), **kw)
        assert f"+silu half={half} " in mpk.describe_program()
    with pytest.raises(_capi.MkError, match="do not divide"):
        mpk = _host_mpk(B=4, R=2)
        mid, wd, y, out = _t(mpk, "mid", 4, 2 * I), _t(mpk, "wd", H, I), mpk.new_tensor((4, H), name="y"), mpk.new_tensor((4, H), name="out")
        mpk.silu_mul_linear_with_residual_layer(input=mid, weight=wd, residual=y, output=out, grid_dim=(H // 64, 1, 1), block_dim=(256, 1, 1), gate_rows_per_group=1000)
        mpk.describe_program()
    # a later reader of the gate/up tensor keeps it written: the activation is a stage of its own
    mpk = _host_mpk(B=4, R=2)
    n, guw = mpk.new_tensor((4, H), name="n"), _t(mpk, "gu", 2 * I, H)
    mid, wd, y, out = mpk.new_tensor((4, 2 * I), name="mid"), _t(mpk, "wd", H, I), mpk.new_tensor((4, H), name="y"), mpk.new_tensor((4, H), name="out")
    mpk.linear_layer(input=n, weight=guw, output=mid, grid_dim=(24, 1, 1), block_dim=(128, 1, 1))
    mpk.silu_mul_linear_with_residual_layer(input=mid, weight=wd, residual=y, output=out, grid_dim=(H // 64, 1, 1), block_dim=(256, 1, 1))
    mpk.silu_mul_layer(input=mid, output=mpk.new_tensor((4, I), name="act"), grid_dim=(1, 1, 1), block_dim=(128, 1, 1))
    kinds = [l.split()[1] for l in mpk.describe_program().splitlines()]
    assert kinds == ["LINEAR", "SILU_MUL", "LINEAR+res", "SILU_MUL"]
    # an input of unknown origin is read as [gate | up] halves by a standalone activation stage
    mpk = _host_mpk(B=4, R=2)
    mid, wd, y, out = _t(mpk, "mid", 4, 2 * I), _t(mpk, "wd", H, I), mpk.new_tensor((4, H), name="y"), mpk.new_tensor((4, H), name="out")
    mpk.silu_mul_linear_with_residual_layer(input=mid, weight=wd, residual=y, output=out, grid_dim=(H // 64, 1, 1), block_dim=(256, 1, 1))
    kinds = [l.split()[1] for l in mpk.describe_program().splitlines()]
    assert kinds == ["SILU_MUL", "LINEAR+res"]
    # a lone split-K linear into a workspace, or a lone reduce, is an error
    mpk = _host_mpk(B=4, R=2)
    mpk.splitk_linear_layer(input=mpk.new_tensor((4, H), name="n"), weight=_t(mpk, "W", H, H),
                            output=mpk.attach_input(torch.zeros(16, H, dtype=torch.float32), "ws"), grid_dim=(8, 4, 1), block_dim=(256, 1, 1))
    with pytest.raises(_capi.MkError, match="must be followed by splitk_reduce_mi300"):
        mpk.describe_program()


def test_layer_methods_that_stand_for_other_tasks():
    """rmsnorm_linear / identity / argmax / attention / *_m_parallel (python/mirage/mpk/persistent_kernel.py:566,587,1953-2043,2153,
    2195): recorded under the reference's task names and ids, lowered to the stages of the tasks they stand for."""
    mpk = _host_mpk(B=4, R=2, max_seq=64, pages=2, page_size=64)
    H, V, D, nq, nkv = 1024, 4096, 128, 8, 2
    x, nw, W = mpk.new_tensor((4, H), name="x"), _t(mpk, "nw", H), _t(mpk, "W", (nq + 2 * nkv) * D, H)
    qkv, att, y, z = mpk.new_tensor((4, (nq + 2 * nkv) * D), name="qkv"), mpk.new_tensor((4, nq * D), name="att"), mpk.new_tensor((4, H), name="y"), mpk.new_tensor((4, H), name="z")
    mpk.rmsnorm_linear_layer(input=x, weight_norm=nw, weight_linear=W, output=qkv, grid_dim=(24, 1, 1), block_dim=(128, 1, 1))
    kc, vc = _t(mpk, "kc", 2, 64, nkv, D), _t(mpk, "vc", 2, 64, nkv, D)
    cos, sin = _t(mpk, "cos", 64, D), _t(mpk, "sin", 64, D)
    mpk.attention_layer(input=qkv, k_cache=kc, v_cache=vc, q_norm=_t(mpk, "qn", D), k_norm=_t(mpk, "kn", D), cos_pos_embed=cos, sin_pos_embed=sin,
                        output=att, grid_dim=(2, nkv, 1), block_dim=(128, 1, 1))
    mpk.linear_with_residual_m_parallel_layer(input=att, weight=_t(mpk, "Wo", H, nq * D), residual=x, output=y, grid_dim=(16, 2, 1), block_dim=(128, 1, 1))
    mpk.identity_layer(input=y, output=z, grid_dim=(1, 1, 1), block_dim=(128, 1, 1))
    lg = mpk.new_tensor((4, V), name="logits")
    mpk.linear_m_parallel_layer(input=z, weight=_t(mpk, "head", V, H), output=lg, grid_dim=(64, 2, 1), block_dim=(128, 1, 1))
    mpk.argmax_layer(input=lg, output=_t(mpk, "tok", 4, 1, dtype=torch.int64), grid_dim=(1, 1, 1), block_dim=(128, 1, 1))
    kinds = [l.split()[1] for l in mpk.describe_program().splitlines()]
    assert kinds == ["NORM[multi-token", "LINEAR+norm", "ATTN", "LINEAR+res", "COPY", "LINEAR", "ARGMAX_PARTIAL", "ARGMAX_REDUCE"], kinds
    tg = json.loads(mpk.kn_graph.generate_task_graph(1, 0)["json_file"])
    types = [t["task_type"] for t in tg["all_tasks"][2:]]
    # TASK_RMS_NORM_LINEAR 102 x24, TASK_ATTENTION_1 103 x4, TASK_LINEAR_WITH_RESIDUAL 108 x32, TASK_IDENTITY 121, TASK_LINEAR 120 x128, TASK_ARGMAX 109
    assert types == [102] * 24 + [103] * 4 + [108] * 32 + [121] + [120] * 128 + [109]
    with pytest.raises(NotImplementedError, match="Blackwell"):
        mpk.tensor_init_layer()


def test_modes_and_configuration_limits():
    meta = make_meta(2, 64, 4, 2, 8, device="cpu")
    kw = dict(world_size=1, mpi_rank=0, num_workers=256, num_local_schedulers=0, num_remote_schedulers=0, max_seq_length=64,
              max_num_batched_requests=2, max_num_batched_tokens=4, max_num_pages=8, page_size=16, meta_tensors=meta, profiler_tensor=None,
              trace_name=None, spec_decode_config=None, use_cutlass_kernel=False)
    for mode in ("offline", "online", "online_notoken", "onepass"):
        assert mi.PersistentKernel(mode=mode, **kw).mode == mode
    for spelling in ("online_multi_turn", "multi_turn"):  # the reference's spelling (persistent_kernel.py:132) and the short one
        with pytest.raises(NotImplementedError, match=spelling):
            mi.PersistentKernel(mode=spelling, **kw)
    with pytest.raises(ValueError, match="Invalid persistent kernel mode"):
        mi.PersistentKernel(mode="sometimes", **kw)
    assert mi.PersistentKernel(mode="offline", **kw).max_tokens_per_request == 8  # the reference's default on AMD
    assert mi.PersistentKernel(mode="offline", max_tokens_per_request=64, **kw).max_tokens_per_request == 64
    with pytest.raises(_capi.MkError, match="max_tokens_per_request"):
        mi.PersistentKernel(mode="offline", max_tokens_per_request=65, **kw)
    # two requests of up to 4 pages each need 8 pages: the page ring hands pages out without checking
    with pytest.raises(_capi.MkError, match="cannot back 2 concurrent requests"):
        mi.PersistentKernel(mode="offline", **{**kw, "max_num_pages": 7, "meta_tensors": make_meta(2, 64, 4, 2, 7, device="cpu")})
    # ... which is a limit of the on-GPU page ring only: where the host owns the page table (online_notoken, onepass) the
    # pool may be oversubscribed, and may hold more pages than the on-GPU scheduler's snapshot could
    for mode in ("online_notoken", "onepass"):
        assert mi.PersistentKernel(mode=mode, **{**kw, "max_num_pages": 5, "meta_tensors": make_meta(2, 64, 4, 2, 5, device="cpu")}).mode == mode
        big = dict(kw, max_num_pages=40000, page_size=1, max_seq_length=64, meta_tensors=make_meta(2, 64, 4, 2, 40000, device="cpu"))
        assert mi.PersistentKernel(mode=mode, **big).mode == mode
    with pytest.raises(_capi.MkError, match="LDS snapshot"):
        mi.PersistentKernel(mode="offline", **dict(kw, max_num_pages=40000, page_size=1, meta_tensors=make_meta(2, 64, 4, 2, 40000, device="cpu")))
    with pytest.raises(_capi.MkError, match="pages per request"):  # the attention stage's own limit holds in every mode
        mi.PersistentKernel(mode="online_notoken", **dict(kw, max_num_pages=40000, page_size=1, max_seq_length=9000,
                                                           meta_tensors=make_meta(2, 9000, 4, 2, 40000, device="cpu")))
    # tensor id -1 is accepted only for the optional operands of the attention tasks
    mpk = _host_mpk()
    x, W = _t(mpk, "x", 4, 1024), _t(mpk, "W", 512, 1024)
    with pytest.raises(_capi.MkError, match="bad tensor id -1"):
        mpk._task("linear", (8, 1, 1), (128, 1, 1), [(x, (-1, -1, -1), 1), (W, (0, -1, -1), 1), (None, (1, -1, -1), -1)])


def test_barrier_counter_comparison_survives_wraparound(tmp_path):
    """The grid barrier compares a 32-bit arrival counter with quota x epoch; both wrap after 2^32 arrivals (about half
    an hour of single-token decode in one launch).  The comparison must stay correct across the wrap."""
    import subprocess
    src = tmp_path / "wrap.cpp"
    src.write_text(r'''
#include <cstdio>
#include <initializer_list>
#include "mk_types.h"
int main() {
  const unsigned quota = 32;
  int bad = 0;
  // epochs around the wrap of quota * epoch (2^27 epochs), and far beyond it
  for (unsigned long long e0 : {1ull, (1ull << 27) - 3, (1ull << 27), (1ull << 28) + 5, (1ull << 32) - 2, (1ull << 33) + 7}) {
    for (unsigned long long e = e0; e < e0 + 6; e++) {
      const unsigned target = quota * (unsigned)e;              // what the kernel computes (wraps)
      const unsigned long long arrived_full = 32ull * e;         // every workgroup has arrived
      for (int missing = 0; missing <= 32; missing += 8) {
        const unsigned counter = (unsigned)(arrived_full - missing);
        const bool expect = missing == 0;
        if (mk_counter_reached(counter, target) != expect) bad++;
      }
      // a die that is already one stage ahead must also read as "reached"
      if (!mk_counter_reached((unsigned)(arrived_full + 32), target)) bad++;
    }
  }
  // the plain comparison is what fails: counter just below 2^32, target wrapped to a small number
  if ((0xFFFFFFE0u >= 0x00000020u) == mk_counter_reached(0xFFFFFFE0u, 0x00000020u)) bad++;
  printf("%d\n", bad);
  return bad != 0;
}
''')
    exe = tmp_path / "wrap"
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fleet-chiplet-megakernel_amd", "csrc")
    subprocess.run(["g++", "-std=c++17", "-O1", "-I", inc, str(src), "-o", str(exe)], check=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True)
    assert res.returncode == 0 and res.stdout.strip() == "0", res.stdout
