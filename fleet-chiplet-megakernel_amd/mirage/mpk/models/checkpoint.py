"""Local checkpoint -> state dict on the GPU, for the model builders.

The reference reaches its weights through `Qwen3ForCausalLM.from_pretrained(model_name)` or, for a local directory,
`load_model(model, f"{model_path}/model{rank}-mp{world_size}.safetensors")` (python/mirage/mpk/models/qwen3/builder.py:
50-66; demo/qwen3/demo.py:197-209), i.e. it instantiates the torch model first and then re-reads its state dict.  Here
the safetensors files are read straight into device tensors under their checkpoint names -- no torch module, no
interleaved copies (the builders make views) -- so loading costs one pass over the files and no extra HBM.

Accepted layouts of `model_path`: a Hugging Face directory (config.json + model.safetensors, or
model.safetensors.index.json + shards), or the reference's per-rank file `model{rank}-mp{world_size}.safetensors`.
Only safetensors files are read (nothing is unpickled).
"""
import json
import os

import torch


def load_config(model_path: str) -> dict:
    with open(os.path.join(model_path, "config.json")) as f:
        return json.load(f)


def _weight_files(model_path: str, rank: int, world_size: int):
    per_rank = os.path.join(model_path, f"model{rank}-mp{world_size}.safetensors")
    if os.path.exists(per_rank):
        return [per_rank]
    index = os.path.join(model_path, "model.safetensors.index.json")
    if os.path.exists(index):
        with open(index) as f:
            shards = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(model_path, s) for s in shards]
    single = os.path.join(model_path, "model.safetensors")
    if os.path.exists(single):
        return [single]
    raise FileNotFoundError(f"no safetensors weights under {model_path} (model.safetensors, model.safetensors.index.json or model{rank}-mp{world_size}.safetensors)")


def load_checkpoint(model_path: str, device="cuda", rank: int = 0, world_size: int = 1, dtype=torch.bfloat16):
    """Returns (config dict, state dict of contiguous `dtype` tensors on `device`)."""
    from safetensors import safe_open
    cfg = load_config(model_path)
    state = {}
    for path in _weight_files(model_path, rank, world_size):
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                t = f.get_tensor(name)
                if t.is_floating_point():
                    t = t.to(dtype)
                state[name] = t.to(device).contiguous()
    need = ["model.embed_tokens.weight", "model.norm.weight"]
    missing = [n for n in need if n not in state]
    if missing:
        raise KeyError(f"checkpoint under {model_path} lacks {missing}")
    return cfg, state


def load_tokenizer(model_path: str):
    """The checkpoint's tokenizer when its files are present and `transformers` is importable, else None (token ids in,
    token ids out still works)."""
    if not any(os.path.exists(os.path.join(model_path, f)) for f in ("tokenizer.json", "tokenizer_config.json", "vocab.json")):
        return None
    try:
        from transformers import AutoTokenizer
        return AutoTokenizer.from_pretrained(model_path, local_files_only=True)
    except Exception:
        return None


def rotary_tables(head_dim: int, theta: float, n_pos: int, device="cuda"):
    """(cos, sin) as the library's rotary module returns them for positions 0..n_pos-1: [1, n_pos, head_dim] bf16, fp32
    math, both halves equal (demo/qwen3/models/modeling_qwen3.py:100-117)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim))
    freqs = torch.arange(n_pos, dtype=torch.float32, device=device)[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(torch.bfloat16)[None].contiguous(), emb.sin().to(torch.bfloat16)[None].contiguous()
