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
    assert (event_no, block, group, ev, typ) == (0, 0, 0, 101, 0) and words[1] >> 32 == 10  # begins at its barrier tick, relative to tick 1000
    event_no, block, group, ev, typ = decode_tag(words[8] & 0xFFFFFFFF, 2, 1)
    assert (event_no, block, group, ev, typ) == (2, 1, 0, 102, 1) and words[8] >> 32 == 960
    out = tmp_path / "t.perfetto-trace"
    kind = export_to_perfetto_trace(buf, str(out))
    assert out.exists()
    if kind == "json":
        tr = json.loads(out.read_text())["traceEvents"]
        slices = [e for e in tr if e["ph"] in ("B", "E")]
        assert len(slices) == 8 and slices[0]["name"] == "TASK_EMBEDDING_0" and slices[0]["pid"] == 0
        assert abs(slices[-1]["ts"] - 9.6) < 1e-9  # 960 ticks = 9.6 us
    # a tensor too small for everything keeps what fits
    small = torch.zeros(4, dtype=torch.uint64)
    assert fill_profiler_tensor(small, profiles) == 2


@pytest.mark.gpu
def test_profiler_tensor_after_a_run(tmp_path):
    from mirage.mpk.profiler_persistent import decode_tag
    from oracle.qwen3_ref import make_model_weights, make_prompt
    from test_qwen3_decode import _decoder, _small_cfg
    cfg = _small_cfg()
    w = make_model_weights(cfg, seed=5)
    dec = _decoder(cfg, w, max_num_batched_tokens=1, max_seq_length=24, page_size=16)
    dec.load_prompts([make_prompt(cfg, 6, 2)])
    dec.mpk.profiler_tensor = torch.zeros(1 << 16, dtype=torch.uint64, device="cuda")
    dec.mpk.trace_name = str(tmp_path / "run")
    dec.mpk()  # one persistent launch; the profile of its last iteration is exported afterwards
    words = dec.mpk.profiler_tensor.cpu().view(torch.int64).tolist()
    st = dec.mpk.stats()
    assert words[0] & 0xFFFFFFFF == st["num_workgroups"] and words[0] >> 32 == 1
    entries = [(decode_tag(wd & 0xFFFFFFFF, st["num_workgroups"], 1), wd >> 32) for wd in words[1:] if wd != 0]
    assert len(entries) >= 2 * st["num_workgroups"] * 5
    # per workgroup and stage: a begin followed by a later end; the linears of the single-token path are among the stages
    open_ = {}
    for (event_no, block, _, ev, typ), ts in entries:
        if typ == 0:
            open_[(block, event_no)] = ts
        else:
            assert ts >= open_.pop((block, event_no))
    assert not open_
    assert {ev for (_, _, _, ev, _), _ in entries} >= {101, 102, 116, 108, 110, 111}
    assert (tmp_path / "run.perfetto-trace").exists() and (tmp_path / "run.pt").exists()
    dec.mpk.finalize()
