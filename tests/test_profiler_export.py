"""The profiler tensor in the reference's (tag, timestamp) entry format and its export for Perfetto
(reference: include/mirage/persistent_kernel/profiler.h:42-54, python/mirage/mpk/profiler_persistent.py:118-165)."""
import json

import pytest
import torch


def test_profiler_tensor_round_trip(tmp_path):
    from mirage.mpk.profiler_persistent import decode_tag, export_to_perfetto_trace, fill_profiler_tensor, stage_event_idx
    assert stage_event_idx("  3 LINEAR+norm+silu rmsnorm_out x w -> y") == 102
    assert stage_event_idx("LINEAR+res a x b") == 108 and stage_event_idx("LINEAR a x b") == 120
    assert stage_event_idx("ATTN attn_in -> attn_out") == 116 and stage_event_idx("ARGMAX_PARTIAL x") == 110
    assert stage_event_idx("MOE_LINEAR+route(single token) x") == 170 and stage_event_idx("MOE_LINEAR silu_mul_out x w2") == 171
    # two workgroups, three stages (one skipped), ticks at 100 MHz
    profiles = [[("  0 EMBED e", 1000, 1010, 1100, 1105), ("  1 NORM[multi-token only] n", 0, 0, 0, 0), ("  2 LINEAR+norm x", 1106, 1200, 1900, 1910)],
                [("  0 EMBED e", 1001, 1012, 1090, 1095), ("  1 NORM[multi-token only] n", 0, 0, 0, 0), ("  2 LINEAR+norm x", 1100, 1201, 1950, 1960)]]
    buf = torch.zeros(64, dtype=torch.uint64)
    n = fill_profiler_tensor(buf, profiles)
    assert n == 8  # begin + end for the two executed stages of each workgroup
    words = buf.view(torch.int64).tolist()
    assert words[0] & 0xFFFFFFFF == 2 and words[0] >> 32 == 1
    event_no, block, group, ev, typ = decode_tag(words[1] & 0xFFFFFFFF, 2, 1)
    assert (event_no, block, group, ev, typ) == (0, 0, 0, 101, 0) and words[1] >> 32 == 100  # begins at its barrier tick, in ns relative to tick 1000
    event_no, block, group, ev, typ = decode_tag(words[8] & 0xFFFFFFFF, 2, 1)
    assert (event_no, block, group, ev, typ) == (2, 1, 0, 102, 1) and words[8] >> 32 == 9600
    out = tmp_path / "t.perfetto-trace"
    kind = export_to_perfetto_trace(buf, str(out))
    assert out.exists()
    if kind == "json":
        tr = json.loads(out.read_text())["traceEvents"]
        slices = [e for e in tr if e["ph"] in ("B", "E")]
        assert len(slices) == 8 and slices[0]["name"] == "TASK_EMBEDDING_0" and slices[0]["pid"] == 0
        assert abs(slices[-1]["ts"] - (9.6 - 0.1)) < 1e-9  # 960 ticks = 9.6 us, counted from the first entry (at 0.1 us)
    # a tensor too small for everything keeps what fits
    small = torch.zeros(4, dtype=torch.uint64)
    assert fill_profiler_tensor(small, profiles) == 2


def test_export_unwraps_the_32_bit_clock(tmp_path):
    """The entries hold the low word of a ns clock (profiler.h:42-54), which wraps every 4.3 s: a recording that crosses
    the wrap exports with times that keep rising within each workgroup."""
    from mirage.mpk.profiler_persistent import encode_tag, export_to_perfetto_trace
    G = 2
    # kernel layout: entry k of workgroup b at 1 + b + k * G; workgroup 1 starts just before the wrap, workgroup 0 after
    raw = {0: [0xFFFFFF00, 0xFFFFFFF0, 0x00000010, 0x00000400], 1: [0xFFFFFE00, 0xFFFFFF80, 0xFFFFFFFF, 0x00000300]}
    buf = torch.zeros(1 + 4 * G, dtype=torch.int64)
    buf[0] = G | (1 << 32)
    for b in range(G):
        for k, ts in enumerate(raw[b]):
            word = encode_tag(k // 2, b, 0, 1, 101 if k < 2 else 102, k & 1) | (ts << 32)
            buf[1 + b + k * G] = word - (1 << 64) if word >= (1 << 63) else word
    out = tmp_path / "w.perfetto-trace"
    if export_to_perfetto_trace(buf.view(torch.uint64), str(out)) != "json":
        pytest.skip("tg4perfetto writes the protobuf form")
    ev = [e for e in json.loads(out.read_text())["traceEvents"] if e["ph"] in ("B", "E")]
    for b in range(G):
        ts = [e["ts"] for e in ev if e["pid"] == b]
        assert ts == sorted(ts) and len(ts) == 4
        assert abs((ts[-1] - ts[0]) * 1000 - ((raw[b][-1] - raw[b][0]) & 0xFFFFFFFF)) < 1e-3  # ns, across the wrap
    # the earliest entry of the buffer (workgroup 1's first) is time zero, workgroup 0 starts 0x100 ns later
    assert min(e["ts"] for e in ev) == 0 and abs(min(e["ts"] for e in ev if e["pid"] == 0) * 1000 - 0x100) < 1e-3


@pytest.mark.gpu
def test_profiler_tensor_records_every_iteration(tmp_path):
    """The kernel itself writes the tensor (profiler.h:129-180): every stage of every iteration, workgroup-interleaved."""
    from mirage.mpk.profiler_persistent import decode_tag
    from oracle.qwen3_ref import make_model_weights, make_prompt
    from test_qwen3_decode import _decoder, _small_cfg
    cfg = _small_cfg()
    w = make_model_weights(cfg, seed=5)
    dec = _decoder(cfg, w, max_num_batched_tokens=1, max_seq_length=24, page_size=16)
    dec.load_prompts([make_prompt(cfg, 6, 2)])
    dec.mpk.profiler_tensor = torch.zeros(1 << 18, dtype=torch.uint64, device="cuda")  # attached after compile
    dec.load_prompts([make_prompt(cfg, 6, 2)])
    dec.mpk.trace_name = str(tmp_path / "run")
    dec.mpk()  # one persistent launch; exported afterwards
    words = dec.mpk.profiler_tensor.cpu().view(torch.int64).tolist()
    st = dec.mpk.stats()
    G, iters = st["num_workgroups"], st["iterations"]
    assert iters >= 10
    assert words[0] & 0xFFFFFFFF == G and words[0] >> 32 == 1
    def after(a, b):  # signed distance a - b of two 32-bit ns timestamps (the clock's low word wraps every 4.3 s)
        return ((a - b + (1 << 31)) & 0xFFFFFFFF) - (1 << 31)

    per_wg = {}
    for i, wd in enumerate(words[1:]):
        if wd == 0:
            continue
        event_no, block, group, ev, typ = decode_tag(wd & 0xFFFFFFFF, G, 1)
        assert block == i % G and group == 0  # entry k of workgroup b sits at 1 + b + k * G
        per_wg.setdefault(block, []).append((event_no, ev, typ, (wd >> 32) & 0xFFFFFFFF))
    assert len(per_wg) == G
    n0 = len(per_wg[0])
    for b, ent in per_wg.items():
        assert len(ent) == n0 and n0 % 2 == 0  # every workgroup passes the same stages
        for k in range(0, n0, 2):
            (e0, ev0, t0, ts0), (e1, ev1, t1, ts1) = ent[k], ent[k + 1]
            assert (e0, ev0, t0, t1) == (e1, ev1, 0, 1) and after(ts1, ts0) >= 0
            if k:
                assert after(ts0, ent[k - 1][3]) >= 0 and 0 < ((e0 - ent[k - 2][0]) & 0x1FFF) < 8  # stages follow one another (skipped ones leave gaps in the numbering)
    # one embedding and one sampling stage per iteration; the fused single-token forms are among the stages
    evs = [e[1] for e in per_wg[0][::2]]
    assert evs.count(101) == iters and evs.count(111) == iters
    assert set(evs) >= {101, 102, 116, 108, 110, 111}
    # a stage's begin on one workgroup is never before the previous stage's end... on the slowest workgroup of that stage is
    # what the barrier gives; checked on whole microseconds of slack for clock skew between dies
    for k in range(2, min(n0, 200), 2):
        base = per_wg[0][k - 2][3]
        assert min(after(per_wg[b][k][3], base) for b in per_wg) + 2000 >= max(after(per_wg[b][k - 2][3], base) for b in per_wg)
    assert (tmp_path / "run.perfetto-trace").exists() and (tmp_path / "run.pt").exists()
    # a tensor that is too small keeps the first entries and nothing is written past its end
    guard = torch.zeros(4 * G + 1 + 64, dtype=torch.uint64, device="cuda")
    dec.mpk.profiler_tensor = guard[:4 * G + 1]
    dec.load_prompts([make_prompt(cfg, 6, 2)])
    dec.mpk()
    gw = guard.cpu().view(torch.int64)
    assert int((gw[1:4 * G + 1] != 0).sum()) == 4 * G and int((gw[4 * G + 1:] != 0).sum()) == 0
    # detached: the kernel records nothing
    dec.mpk.profiler_tensor = None
    guard.zero_()
    dec.load_prompts([make_prompt(cfg, 6, 2)])
    dec.mpk()
    assert int((guard.cpu().view(torch.int64) != 0).sum()) == 0
    dec.mpk.finalize()
