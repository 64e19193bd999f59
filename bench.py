"""Headline benchmark: decode TPOT (ms/token) of the 36-layer Qwen3-8B-shaped random-init bf16 model on one MI355X.

A "step" is one decode iteration of the persistent megakernel for the whole batch.  The prompt (80 seeded random ids
per request) is ingested and W warm-up decode steps run untimed; then EXACTLY K decode steps run inside ONE persistent
launch, bracketed by torch.cuda.synchronize() on both sides.  Weights, KV cache and meta tensors are resident in HBM
before the timed region.  Prints one JSON line.  The metric is quoted at two batch sizes: the default run times BS=1
(the line's `value`, `ms_per_step`, `roofline`) and then BS=64 on the same weights (the line's "bs64" object, with its
own ms_per_step, context range and roofline); --batch N runs one batch size only.

roofline: the dominant (only) kernel is mk_persistent_kernel; its algorithmic bytes per launch are
K x (all bf16 weight matrices once + the K/V rows of every cached position of every request), divided by the launch
duration measured with HIP events on the launch stream, against the 8 TB/s HBM peak.
cpu_baseline: the CPU oracle's torch-order decode (the reference's PyTorch path restated) of the whole model timed on the
host cores: an 80-token prompt, then a window of 8 decode steps (a few layers + LM head extrapolated when the host has
too little memory for the 16 GB of weights); a reported baseline, not a target.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "fleet-chiplet-megakernel_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def cpu_baseline(shape, window=8, prompt_len=80):
    """The oracle's torch-order decode (the reference's PyTorch path restated) of the WHOLE model on the host cores: an
    80-token prompt, then a window of `window` greedy decode steps, timed step by step.  The weights are one random layer
    copied into distinct memory for every layer (16 GB for the 8B shape; timing depends on shapes and on streaming distinct
    memory, not on the values).  With less than 40 GB of free host memory the few-layer extrapolation below is used."""
    import torch
    avail = None
    try:
        import psutil
        avail = psutil.virtual_memory().available
    except Exception:
        pass
    if shape.num_experts > 0 or avail is None or avail < 40 * (1 << 30):
        return cpu_baseline_extrapolated(shape)
    from oracle.qwen3_ref import KVCache, Qwen3Config, Qwen3Oracle, make_layer_weights
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    cfg = Qwen3Config(hidden_size=shape.hidden_size, num_q_heads=shape.num_q_heads, num_kv_heads=shape.num_kv_heads, head_dim=shape.head_dim,
                      intermediate_size=shape.intermediate_size, num_layers=shape.num_layers, vocab_size=shape.vocab_size, rope_theta=shape.rope_theta)
    g = torch.Generator().manual_seed(0)
    one = make_layer_weights(cfg, g)
    w = {"layers": [one] + [{k: v.clone() for k, v in one.items()} for _ in range(cfg.num_layers - 1)]}
    blk = (torch.randn(4096, cfg.hidden_size, generator=g) * 0.02).to(torch.bfloat16)
    reps = math.ceil(cfg.vocab_size / 4096)
    w["embed"] = blk.repeat(reps, 1)[:cfg.vocab_size].contiguous()
    w["lm_head"] = blk.flip(0).repeat(reps, 1)[:cfg.vocab_size].contiguous()
    w["final_norm"] = torch.ones(cfg.hidden_size, dtype=torch.bfloat16)
    orc = Qwen3Oracle(cfg, w, "torch")
    cache = KVCache(cfg, prompt_len + window + 2)
    prompt = torch.randint(0, cfg.vocab_size, (prompt_len,), generator=torch.Generator().manual_seed(0))
    t0 = time.perf_counter()
    tok = orc.forward(prompt, cache, 0)[-1].argmax(-1).view(1)  # prefill (also the warm-up)
    t_prefill = time.perf_counter() - t0
    per_step = []
    for s in range(window):
        t0 = time.perf_counter()
        tok = orc.forward(tok, cache, prompt_len + s)[-1].argmax(-1).view(1)
        per_step.append(time.perf_counter() - t0)
    ms = sum(per_step) / window * 1e3
    return {"value": round(ms, 2), "unit": "ms/token", "cores": cores, "kind": "port",
            "sample": f"BS=1, whole {shape.num_layers}-layer model + LM head: {prompt_len}-token prompt ({t_prefill:.1f} s), then a window of {window} greedy decode "
                      f"steps, mean per step (min {min(per_step) * 1e3:.1f}, max {max(per_step) * 1e3:.1f} ms); torch-order bf16 oracle, {cores} threads"}


def cpu_baseline_extrapolated(shape, n_layers_sample=2, steps=3, context=80):
    """Fallback when the whole model does not fit the host: `n_layers_sample` full-width layers + LM head, extrapolated."""
    import torch
    from oracle.qwen3_ref import KVCache, Qwen3Config, Qwen3Oracle, make_layer_weights
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    cfg = Qwen3Config(hidden_size=shape.hidden_size, num_q_heads=shape.num_q_heads, num_kv_heads=shape.num_kv_heads, head_dim=shape.head_dim,
                      intermediate_size=shape.intermediate_size, num_layers=n_layers_sample, vocab_size=shape.vocab_size, rope_theta=shape.rope_theta,
                      num_experts=shape.num_experts, num_experts_per_tok=shape.num_experts_per_tok, moe_intermediate_size=shape.moe_intermediate_size)
    g = torch.Generator().manual_seed(0)
    w = {"layers": [make_layer_weights(cfg, g) for _ in range(n_layers_sample)]}
    w["embed"] = torch.zeros(8, cfg.hidden_size, dtype=torch.bfloat16)
    w["embed"][:] = torch.randn(8, cfg.hidden_size, generator=g).to(torch.bfloat16) * 0.02
    w["final_norm"] = torch.ones(cfg.hidden_size, dtype=torch.bfloat16)
    # LM head: reuse one 4096-row random block 37x + remainder to bound the generation time; timing only depends on shape
    blk = (torch.randn(4096, cfg.hidden_size, generator=g) * 0.02).to(torch.bfloat16)
    reps = math.ceil(cfg.vocab_size / 4096)
    w["lm_head"] = blk.repeat(reps, 1)[:cfg.vocab_size].contiguous()
    orc = Qwen3Oracle(cfg, w, "torch")
    cache = KVCache(cfg, context + steps + 2)
    cache.k.normal_(0, 1, generator=g)
    cache.v.normal_(0, 1, generator=g)
    ids = torch.tensor([1])

    def layers_only(pos):
        x = w["embed"][ids]
        for li in range(cfg.num_layers):
            x = orc.layer(li, x, cache, pos)
        return x

    def head_only(x):
        from oracle.qwen3_ref import rmsnorm_t
        import torch.nn.functional as F
        return F.linear(rmsnorm_t(x, w["final_norm"]), w["lm_head"]).argmax(-1)

    x = layers_only(context)  # warm-up
    head_only(x)
    t_layers, t_head = [], []
    for s in range(steps):
        t0 = time.perf_counter()
        x = layers_only(context + s)
        t1 = time.perf_counter()
        head_only(x)
        t2 = time.perf_counter()
        t_layers.append((t1 - t0) / n_layers_sample)
        t_head.append(t2 - t1)
    per_layer = sorted(t_layers)[len(t_layers) // 2]
    head = sorted(t_head)[len(t_head) // 2]
    ms = (per_layer * shape.num_layers + head) * 1e3
    return {"value": round(ms, 2), "unit": "ms/token", "cores": cores, "kind": "port",
            "sample": f"BS=1, context {context}: {n_layers_sample} of {shape.num_layers} full-width layers + LM head, median of {steps} steps, "
                      f"extrapolated to {shape.num_layers} layers; torch-order bf16 oracle"}


# HBM bytes as the counters saw them (rocprofv3 --pmc FETCH_SIZE x 2.0 + WRITE_SIZE, both scaled by a 1 GiB copy in the same
# run; the passes and their commands are in profiles/mk_persistent_kernel_qwen3-8b_bs1.md and ..._bs64.md).  Counter
# passes cannot run inside a timed benchmark, so the bench line derives its `traffic` from those passes: the measured
# bytes of the profiled 1024-step launch minus that launch's K/V rows (which are read exactly once: the counters show no
# excess at BS=1, where K/V is all there is besides the weights) give the per-step part -- weights, activations,
# K-slice partials written and read back --, and the K/V rows of THIS launch's contexts are added to it.  A model, depth
# or batch size without a committed counter pass reports null.
MEASURED_PER_STEP_BYTES_EXCL_KV = {("qwen3-8b", 36, 1): (15.6246e12 + 15.75e9 - 623104 * 147456) / 1024,
                                   ("qwen3-8b", 36, 64): (25.9037e12 + 1.4046e12 - (24191940165632 - 1024 * 15136194560)) / 1024}


def print_stage_profile(dec, B, out=sys.stderr):
    """Where the last iteration of the last launch went: per stage, over all workgroups, when they entered the stage, when
    they saw the previous stage's barrier complete and when they arrived at the stage's own barrier (microseconds after
    the first workgroup entered the first stage; device timestamps, 100 MHz)."""
    import numpy as np
    G = dec.mpk.stats()["num_workgroups"]
    prof = [dec.mpk.stage_profile(w, raw=True) for w in range(G)]
    rows = [i for i in range(len(prof[0]) - 1) if prof[0][i][1] > 0]  # (the last record times the scheduler step)
    t0 = min(prof[w][rows[0]][1] for w in range(G))
    print(f"stage profile, BS={B}, last iteration ({G} workgroups; us): entered min..max | barrier seen min..max | arrived min / median / max", file=out)
    for i in rows:
        ent, seen, arr = (np.array([prof[w][i][k] for w in range(G)], dtype=np.float64) * 0.01 - t0 * 0.01 for k in (1, 2, 4))
        print(f"  {prof[0][i][0][:56]:56s} {ent.min():8.1f}..{ent.max():8.1f} | {seen.min():8.1f}..{seen.max():8.1f} | "
              f"{arr.min():8.1f} / {np.median(arr):8.1f} / {arr.max():8.1f}", file=out)
    out.flush()


def run_leg(torch, dec, shape, model, B, K, W, P, max_seq, mode, stage_profile=False):
    """Ingest B prompts of P tokens, run W untimed decode steps, then time exactly K decode steps in ONE persistent launch."""
    prompts = [torch.randint(0, shape.vocab_size, (P,), generator=torch.Generator().manual_seed(r)) for r in range(B)]
    dec.load_prompts(prompts)
    # prompt ingestion: run until every request has consumed its prompt (first decode token produced), then warm up
    prefill_iters = 0
    while True:
        dec.mpk.run_steps(1)
        prefill_iters += 1
        if int(dec.meta["step"].min().item()) >= P:
            break
        assert prefill_iters < 10 * P * B, "prompt ingestion did not finish"
    if W > 0:
        dec.mpk.run_steps(W)
    steps0 = dec.meta["step"].cpu().tolist()   # cached positions of every request at the first timed step (requests that
    ctx0, ctx0_max = min(steps0), max(steps0)  # ingested their prompt earlier are further along: prompts enter 8 requests at a time)
    stream = torch.cuda.current_stream()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.mpk.enqueue_steps(K, default_stream=stream)
    finished = dec.mpk.wait(default_stream=stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    st = dec.mpk.stats()
    assert not finished, "requests finished inside the timed region; lower --steps"
    steps1 = dec.meta["step"].cpu().tolist()
    assert steps1 == [s0 + K for s0 in steps0], f"timed region did not run exactly K={K} decode steps for every request: {steps0} -> {steps1}"
    if stage_profile:
        print_stage_profile(dec, B)
    wall_ms = (t1 - t0) * 1e3
    kernel_ms = st["last_launch_ms"]
    ms_per_step = wall_ms / K
    # algorithmic bytes: weights once per step + K/V rows of every cached position (positions ctx0+1 .. ctx0+K incl. the new one)
    kv_positions = sum(s0 + 1 + i for s0 in steps0 for i in range(K))  # summed over the requests
    # mixture of experts: a step streams the experts its tokens select; B tokens choosing top-k of E uniformly touch
    # E * (1 - (1 - k/E)^B) distinct experts per layer in expectation (exactly k for one token)
    moe = shape.num_experts > 0
    distinct = None
    if moe and B > 1:
        distinct = shape.num_experts * (1.0 - (1.0 - shape.num_experts_per_tok / shape.num_experts) ** B)
    bytes_total = int(K * shape.weight_bytes_per_token(distinct) + kv_positions * shape.kv_bytes_per_position())
    achieved = bytes_total / (kernel_ms * 1e-3) / 1e9
    per_step = MEASURED_PER_STEP_BYTES_EXCL_KV.get((model, shape.num_layers, B))
    traffic = None if per_step is None else int(per_step * K + kv_positions * shape.kv_bytes_per_position())
    return {
        "batch": B, "ms_per_step": round(ms_per_step, 4), "tokens_per_s": round(B * 1e3 / ms_per_step, 1), "steps": K, "warmup": W,
        "workload": f"{'Qwen3-30B-A3B (128 experts, top-8)' if moe else 'Qwen3-8B'} shape, {shape.num_layers} layers, vocab {shape.vocab_size}, BS={B}, prompt {P}, "
                    f"context {ctx0}..{ctx0_max + K}, max_seq_len {max_seq}, page_size 4096, graph mode {mode}",
        "prefill_iterations": prefill_iters,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": traffic,
                     "traffic_source": None if per_step is None else "FETCH_SIZE/WRITE_SIZE counter passes of the 1024-step launch in profiles/: its per-step bytes other than K/V rows x this launch's steps + this launch's K/V rows",
                     "kernel": "mk_persistent_kernel_m1" if B == 1 else "mk_persistent_kernel", "kernel_ms_per_launch": round(kernel_ms, 3), "algorithmic_bytes_per_launch": bytes_total},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1024)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=None,
                    help="requests decoded concurrently (BS).  Default: the metric's two batch sizes, 1 (the headline `value`) and 64 (reported under \"bs64\")")
    ap.add_argument("--layers", type=int, default=36)
    ap.add_argument("--prompt-length", type=int, default=80)
    ap.add_argument("--mode", choices=["fleet", "mpk"], default="fleet")
    ap.add_argument("--model", choices=["qwen3-8b", "qwen3-30b-a3b"], default="qwen3-8b",
                    help="qwen3-8b: the headline dense shape; qwen3-30b-a3b: the mixture-of-experts shape (128 experts, top-8), reported alongside")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--single-weight-copy", action="store_true",
                    help="keep every linear weight once, in matrix-core tile order (BS >= 2): what the memory saving costs iterations of one or two tokens")
    ap.add_argument("--calib-copy", action="store_true", help="also run one 1 GiB device-to-device copy (scale for rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--stage-profile", action="store_true",
                    help="after each timed launch, print its last iteration's per-stage timeline over all workgroups to stderr")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the decode megakernel on ONE GPU; --gpus must be 1 "
              "(multi-GPU tensor parallelism is not built)", file=sys.stderr)
        sys.exit(2)
    if int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: launched with WORLD_SIZE>1; this benchmark is single-GPU", file=sys.stderr)
        sys.exit(2)
    import torch
    from demo_qwen3 import Qwen3Decoder, Qwen3Shape, random_weights
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the megakernel has no CPU path", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    from mirage import _capi
    # where the library is mapped (a crash report of the process can be matched against it)
    print(f"bench.py: pid {os.getpid()}, {_capi.LIB_PATH} at {_capi.load_address():#x}", file=sys.stderr, flush=True)
    moe = args.model == "qwen3-30b-a3b"
    shape = Qwen3Shape.qwen3_30b_a3b(min(args.layers, 48) if args.layers != 36 else 48) if moe else Qwen3Shape(num_layers=args.layers)
    K, W, P = args.steps, args.warmup, args.prompt_length
    batches = [args.batch] if args.batch else ([1, 64] if not moe else [1])
    if args.calib_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    weights = random_weights(shape, seed=0)
    legs = []
    for B in batches:
        # The on-GPU scheduler shares B token slots per iteration between decoding requests (one each) and prompt ingestion
        # (8 tokens per request), exactly as the reference's does: at B = 64 the first requests have decoded some 360 tokens
        # by the time the last one has ingested its prompt.  The timed K steps start once ALL B requests decode, so the
        # requests sit at different contexts (the range is in `workload`; the KV bytes of the roofline are the real ones);
        # max_seq_len is the configuration's 1200 unless the earliest request's K timed steps would not fit.
        max_seq = max(1200, P + W + K + 2 + (0 if B == 1 else 6 * P))
        dec = Qwen3Decoder(shape, weights, max_num_batched_tokens=B, max_num_batched_requests=B, max_seq_length=max_seq, page_size=4096, mode=args.mode,
                           single_weight_copy=args.single_weight_copy)
        legs.append(run_leg(torch, dec, shape, args.model, B, K, W, P, max_seq, args.mode, args.stage_profile))
        dec.mpk.finalize()
        del dec
    del weights
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    head = legs[0]
    name = "Qwen3-30B-A3B" if moe else "Qwen3-8B"
    out = {
        "metric": f"decode TPOT ms/token @BS={','.join(str(l['batch']) for l in legs)} {name}-shape bf16; % of HBM roofline",
        "value": head["ms_per_step"], "unit": "ms/token", "n_gpus": 1, "steps": K,
        "warmup": W, "ms_per_step": head["ms_per_step"], "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (random-init weights ~N(0,0.02), seeded random prompts)",
        "config": {"workload": head["workload"], "batch": head["batch"], "tokens_per_s": head["tokens_per_s"], "prefill_iterations": head["prefill_iterations"]},
        "roofline": head["roofline"],
    }
    for leg in legs[1:]:
        out[f"bs{leg['batch']}"] = leg  # the metric's other batch size: same model, same steps, its own roofline
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(shape)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
