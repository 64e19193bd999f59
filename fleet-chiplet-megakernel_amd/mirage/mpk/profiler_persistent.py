"""Device timeline of the persistent kernel in the reference's profiler-buffer format, and its export for Perfetto.

The reference's kernels write (tag, timestamp) entries into a caller-supplied uint64 tensor when a profiler tensor is
passed (include/mirage/persistent_kernel/profiler.h:42-54,129-180) and `PersistentKernel.__call__` turns it into a
Perfetto trace afterwards (python/mirage/mpk/persistent_kernel.py:2644-2658, python/mirage/mpk/profiler_persistent.py).
Here the kernel does the same once the tensor is attached (mk_set_profiler; `PersistentKernel(profiler_tensor=...)` does
it at compile time): begin and end of every stage each workgroup executes, every iteration, until the tensor is full.
Independently of that the kernel always keeps finer per-stage ticks of the LAST iteration (mk_get_stage_profile), and
`fill_profiler_tensor` re-expresses those in the same entry format for a tensor that was not attached:

    entry 0            : int32 pair (num_blocks, num_groups)
    entry i (non-zero) : low 32 bits  tag = event_no << 19 | (block * num_groups + group) << 11 | event_idx << 2 | type
                         high 32 bits timestamp in ns (low word of the 100 MHz device clock x 10, as the reference keeps the low word
                         of its ns timer; fill_profiler_tensor counts from the iteration's earliest tick)
    type               : 0 begin, 1 end, 2 instant; event_idx is the reference's task-type number of the stage

`export_to_perfetto_trace` decodes such a tensor.  With the `tg4perfetto` package (what the reference uses; not present in
this environment) it writes the same protobuf trace; without it, the Chrome trace-event JSON that ui.perfetto.dev opens
as well -- one process per workgroup ("block_<n>"), one slice per stage."""
import json

import torch

# the reference's task-type numbers (profiler_persistent.py:11-106) for the stage kinds of the stage program
STAGE_EVENT = (
    ("EMBED", 101, "TASK_EMBEDDING"), ("NORM", 119, "TASK_RMS_NORM"), ("LINEAR+norm", 102, "TASK_RMS_NORM_LINEAR"),
    ("LINEAR+res", 108, "TASK_LINEAR_WITH_RESIDUAL"), ("LINEAR", 120, "TASK_LINEAR"), ("SILU_MUL", 118, "TASK_SILU_MUL"),
    ("ATTN", 116, "TASK_PAGED_ATTENTION_1"), ("MOE_TOPK", 172, "TASK_MOE_TOPK_SOFTMAX_MI300"), ("MOE_LINEAR+route", 170, "TASK_MOE_W13_LINEAR_MI300"),
    ("MOE_LINEAR+silu", 170, "TASK_MOE_W13_LINEAR_MI300"), ("MOE_LINEAR", 171, "TASK_MOE_W2_LINEAR_MI300"), ("MOE_COMBINE", 173, "TASK_MOE_MUL_SUM_ADD_MI300"),
    ("ARGMAX_PARTIAL", 110, "TASK_ARGMAX_PARTIAL"), ("ARGMAX_REDUCE", 111, "TASK_ARGMAX_REDUCE"), ("SCHEDULER", 200, "TASK_SCHD_TASKS"))
EVENT_NAMES = {idx: name for _, idx, name in STAGE_EVENT}


def stage_event_idx(description: str) -> int:
    """Task-type number for a stage description line ("LINEAR+norm+silu rmsnorm_out x ... ")."""
    words = description.split()
    if words and words[0].isdigit():  # listing lines carry the stage number in front
        words = words[1:]
    head = words[0] if words else ""
    best = (0, 121)  # TASK_IDENTITY for anything unknown
    for prefix, idx, _ in STAGE_EVENT:
        if head.startswith(prefix) and len(prefix) > best[0]:
            best = (len(prefix), idx)
    return best[1]


def encode_tag(event_no: int, block: int, group: int, num_groups: int, event_idx: int, event_type: int) -> int:
    return ((event_no & 0x1FFF) << 19) | (((block * num_groups + group) & 0xFF) << 11) | ((event_idx & 0x1FF) << 2) | (event_type & 0x3)


def decode_tag(tag: int, num_blocks: int, num_groups: int):
    block_group = (tag >> 11) & 0xFF
    return tag >> 19, block_group // num_groups, block_group % num_groups, (tag >> 2) & 0x1FF, tag & 0x3


def fill_profiler_tensor(profiler_tensor: torch.Tensor, profiles, num_groups: int = 1) -> int:
    """profiles[w] = list of (description, entered, barrier_satisfied, work_done, arrived) in 100 MHz ticks for workgroup w
    (PersistentKernel.stage_profile(w, raw=True); 0 = stage skipped).  Writes a begin entry at `barrier_satisfied` (when the
    stage's own work starts) and an end entry at `arrived` per executed stage, workgroup-major, as many as fit.  The 8-bit
    block field of the format holds 256 workgroups.  Returns the number of entries written (the header not counted)."""
    assert profiler_tensor.dtype in (torch.uint64, torch.int64) and profiler_tensor.dim() == 1
    cap = profiler_tensor.numel() - 1
    ticks = [p[i] for prof in profiles for p in prof for i in (1, 2, 3, 4) if p[i] > 0]
    t0 = min(ticks) if ticks else 0
    words = [len(profiles) | (num_groups << 32)]
    for w, prof in enumerate(profiles):
        for s, p in enumerate(prof):
            begin, end = (p[2] if p[2] > 0 else p[1]), (p[4] if p[4] > 0 else p[3])
            if p[0].split() and p[0].split()[-1] == "SCHEDULER":  # (previous iteration complete, prepared, published, -)
                begin, end = p[1], p[3]
            if begin <= 0 or end <= 0 or len(words) + 1 > cap:
                continue
            ev = stage_event_idx(p[0])
            words.append(encode_tag(s, w, 0, num_groups, ev, 0) | ((((begin - t0) * 10) & 0xFFFFFFFF) << 32))
            words.append(encode_tag(s, w, 0, num_groups, ev, 1) | ((((end - t0) * 10) & 0xFFFFFFFF) << 32))
    host = torch.zeros(profiler_tensor.numel(), dtype=torch.int64)
    # (values above 2^63 do not occur: timestamps are relative and below 2^31 for any iteration shorter than 2 s)
    host[:len(words)] = torch.tensor(words, dtype=torch.int64)
    profiler_tensor.copy_(host.view(profiler_tensor.dtype) if profiler_tensor.dtype != torch.int64 else host)
    return len(words) - 1


def export_to_perfetto_trace(profiler_buffer: torch.Tensor, file_name: str) -> str:
    """Decode a profiler tensor (the format above) and write a trace Perfetto opens.  Returns "protobuf" or "json"."""
    words = profiler_buffer.cpu().view(torch.int64).tolist()
    num_blocks, num_groups = words[0] & 0xFFFFFFFF, max(1, (words[0] >> 32) & 0xFFFFFFFF)
    entries = []
    for wd in words[1:]:
        if wd == 0:
            continue
        tag, ts = wd & 0xFFFFFFFF, (wd >> 32) & 0xFFFFFFFF
        entries.append(decode_tag(tag, num_blocks, num_groups) + (ts,))
    # The timestamps are the low 32 bits of a ns clock and wrap every 4.3 s.  Within a workgroup time only moves forward
    # (entries are in the order they were written), so each workgroup's sequence is unwrapped by its forward differences;
    # its first entry is placed by its signed 32-bit distance to the first entry of the buffer.
    ref, last, unwrapped = None, {}, []
    for e in entries:
        ts, key = e[5], (e[1], e[2])
        if ref is None:
            ref = ts
        if key in last:
            prev_raw, prev_t = last[key]
            t = prev_t + ((ts - prev_raw) & 0xFFFFFFFF)
        else:
            t = ((ts - ref + (1 << 31)) & 0xFFFFFFFF) - (1 << 31)
        last[key] = (ts, t)
        unwrapped.append(e[:5] + (t,))
    # entries of one workgroup in time order (begin before end on equal times); times count from the earliest
    t0 = min((e[5] for e in unwrapped), default=0)
    entries = sorted((e[:5] + (e[5] - t0,) for e in unwrapped), key=lambda e: (e[1], e[2], e[5], e[0], e[4]))
    try:
        from tg4perfetto import TraceGenerator  # the reference's writer
    except ImportError:
        TraceGenerator = None
    if TraceGenerator is not None:
        tgen = TraceGenerator(file_name)
        groups = {}
        for b in range(num_blocks):
            pid = tgen.create_group(f"block_{b}")
            for g in range(num_groups):
                groups[(b, g)] = pid.create_group(f"group_{g}")
        tracks = {}
        for event_no, b, g, ev, typ, ts in entries:
            key = (b, g, ev)
            if key not in tracks:
                tracks[key] = groups[(b, g)].create_track()
            name = f"{EVENT_NAMES.get(ev, 'TASK_' + str(ev))}_{event_no}"
            if typ == 0:
                tracks[key].open(ts, name)
            elif typ == 1:
                tracks[key].close(ts)
            else:
                tracks[key].instant(ts, name)
        tgen.flush()
        return "protobuf"
    events = []
    for b in range(num_blocks):
        events.append({"ph": "M", "name": "process_name", "pid": b, "args": {"name": f"block_{b}"}})
    for event_no, b, g, ev, typ, ts in entries:
        name = f"{EVENT_NAMES.get(ev, 'TASK_' + str(ev))}_{event_no}"
        events.append({"ph": "B" if typ == 0 else ("E" if typ == 1 else "i"), "name": name, "pid": b, "tid": g, "ts": ts * 0.001})  # ns -> us
    with open(file_name, "w") as f:
        json.dump({"traceEvents": events, "displayTimeUnit": "ns"}, f)
    return "json"
