"""Shared builders for the parity tests: meta tensors, PersistentKernel construction, and the Qwen3 decode graph
expressed through the PersistentKernel layer API exactly as demo/qwen3/demo.py:314-1169 does."""
import os

import torch

import mirage as mi


def make_meta(total_requests, max_seq, max_tokens, max_requests, max_pages, device="cuda"):
    return {
        "step": torch.zeros(total_requests, dtype=torch.int32, device=device),
        "tokens": torch.zeros(total_requests, max_seq, dtype=torch.int64, device=device),
        "input_tokens": torch.zeros(max_tokens, 1, dtype=torch.int64, device=device),
        "output_tokens": torch.zeros(max_tokens, 1, dtype=torch.int64, device=device),
        "num_new_tokens": torch.ones(total_requests, dtype=torch.int32, device=device),
        "prompt_lengths": torch.zeros(total_requests, dtype=torch.int32, device=device),
        "qo_indptr_buffer": torch.zeros(max_requests + 1, dtype=torch.int32, device=device),
        "paged_kv_indptr_buffer": torch.zeros(max_requests + 1, dtype=torch.int32, device=device),
        "paged_kv_indices_buffer": torch.zeros(max_pages, dtype=torch.int32, device=device),
        "paged_kv_last_page_len_buffer": torch.zeros(max_requests, dtype=torch.int32, device=device),
    }


def make_mpk(meta, max_seq, max_tokens, max_requests, max_pages, page_size, mode="offline", eos=0x7FFFFFFF, num_workers=None):
    if num_workers is None:
        num_workers, _ = mi.get_configurations_from_gpu(0)
    return mi.PersistentKernel(
        mode=mode, world_size=1, mpi_rank=0, num_workers=num_workers, num_local_schedulers=0, num_remote_schedulers=0,
        max_seq_length=max_seq, max_num_batched_requests=max_requests, max_num_batched_tokens=max_tokens,
        max_num_pages=max_pages, page_size=page_size, eos_token_id=eos, meta_tensors=meta, profiler_tensor=None,
        trace_name=None, spec_decode_config=None, use_cutlass_kernel=False)


def bf16_ulp_diff(a, b, floor=1e-30):
    """Max difference in units of bf16 ulp of the larger magnitude (magnitudes below `floor` count as `floor`, so
    cancellation near zero is measured against the scale of the operands), plus max abs diff."""
    af, bf = a.float().cpu(), b.float().cpu()
    d = (af - bf).abs()
    scale = torch.maximum(af.abs(), bf.abs()).clamp_min(floor)
    ulp = torch.exp2(torch.floor(torch.log2(scale)) - 7)
    return float((d / ulp).max()), float(d.max())
