"""The serving-facing wrapper (mirage.mpk.MPK + MPKMetadata) and the Qwen3 graph builder on a small random model
(reference: python/mirage/mpk/mpk.py:16-428, python/mirage/mpk/models/qwen3/builder.py:13-824).

* host only (no GPU): the builder's task sequence -- rmsnorm, split-K linear + reduce, paged attention, linear,
  silu_mul_linear_with_residual, LM head, argmax -- records, validates and lowers to the stage program;
* GPU, build_from_config: offline generation equals the layer-API driver's on the same weights and passes the
  teacher-forced oracle check (the first-tokens criterion of tests/ci-tests/test_inference_output.py:23-43);
* GPU, build_from_model: a local safetensors checkpoint directory (config.json + model.safetensors) gives the same tokens;
* GPU, online_notoken without LM head: one pass returns the normalised final hidden state (mpk.py:419-421)."""
import json
import os

import pytest
import torch


def _cfg(layers=2, vocab=2048):
    from oracle.qwen3_ref import Qwen3Config
    return Qwen3Config(hidden_size=1024, num_q_heads=8, num_kv_heads=2, head_dim=128, intermediate_size=1536, num_layers=layers, vocab_size=vocab)


def _state_dict(w, device):
    """Oracle weights under the checkpoint's names."""
    sd = {"model.embed_tokens.weight": w["embed"], "model.norm.weight": w["final_norm"], "lm_head.weight": w["lm_head"]}
    names = {"input_norm": "input_layernorm.weight", "q_proj": "self_attn.q_proj.weight", "k_proj": "self_attn.k_proj.weight",
             "v_proj": "self_attn.v_proj.weight", "q_norm": "self_attn.q_norm.weight", "k_norm": "self_attn.k_norm.weight",
             "o_proj": "self_attn.o_proj.weight", "post_norm": "post_attention_layernorm.weight", "gate_proj": "mlp.gate_proj.weight",
             "up_proj": "mlp.up_proj.weight", "down_proj": "mlp.down_proj.weight"}
    for i, lw in enumerate(w["layers"]):
        for k, n in names.items():
            sd[f"model.layers.{i}.{n}"] = lw[k]
    return {k: v.to(device).contiguous() for k, v in sd.items()}


def _metadata(cfg, w, device, mode="offline", R=3, T=8, total=5, max_seq=40, PS=16, with_lm_head=True, from_path=None, num_workers=-1):
    from mirage.mpk import MirageModelConfig, MPKMetadata
    from oracle.qwen3_ref import rope_tables
    pages = R * ((max_seq + PS - 1) // PS)
    md = MPKMetadata(mode=mode, total_num_requests=total, max_seq_length=max_seq, max_num_batched_requests=R, max_num_batched_tokens=T,
                     max_num_pages=pages, page_size=PS, device=device, eos_token_id=0x7FFFFFFF, num_workers=num_workers, num_schedulers=0)
    if from_path is not None:
        md.weight_from_model, md.model_path, md.model_name = True, from_path, "Qwen3"
        return md
    cos, sin = rope_tables(cfg, max(max_seq, 16))
    shape = (cfg.num_layers, pages, PS, cfg.num_kv_heads, cfg.head_dim)
    md.model_config = MirageModelConfig(
        hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size, vocab_size=cfg.vocab_size, local_num_q_heads=cfg.num_q_heads,
        local_num_kv_heads=cfg.num_kv_heads, head_dim=cfg.head_dim, num_layers=cfg.num_layers,
        k_cache=torch.zeros(shape, dtype=torch.bfloat16, device=device), v_cache=torch.zeros(shape, dtype=torch.bfloat16, device=device),
        position_embeddings=(cos[None].to(device), sin[None].to(device)), state_dict=_state_dict(w, device), with_lm_head=with_lm_head)
    return md


def _load_prompts(mpk, prompts):
    mpk.tokens.zero_()
    mpk.prompt_lengths.zero_()
    for r, p in enumerate(prompts):
        mpk.tokens[r, :len(p)].copy_(p.to(mpk.tokens.device))
        mpk.prompt_lengths[r] = len(p)
    mpk.step.zero_()


def test_builder_task_sequence_lowers_on_the_host():
    """No GPU: CPU meta tensors make a host-only graph; the builder's tasks must validate and lower."""
    from mirage.mpk import MPK
    from oracle.qwen3_ref import make_model_weights
    cfg = _cfg()
    w = make_model_weights(cfg, seed=61)
    mpk = MPK(_metadata(cfg, w, "cpu", num_workers=256))
    mpk.build()
    res = mpk.generate_task_graph()
    tg = json.loads(open(res["json_file"]).read()) if os.path.exists(str(res.get("json_file", ""))) else None
    prog = mpk.persistent_kernel.describe_program()
    lines = [l for l in prog.splitlines() if l.strip()]
    ops = [l.split()[1] if l.split()[0].isdigit() else l.split()[0] for l in lines]
    per_layer = ["LINEAR+norm", "ATTN", "LINEAR+res", "NORM[multi-token", "LINEAR+norm+silu", "LINEAR+res", "NORM[multi-token"]
    assert sum(o.startswith("ATTN") for o in ops) == cfg.num_layers
    assert sum(o.startswith("LINEAR") for o in ops) == 4 * cfg.num_layers + 1, prog
    assert any(o.startswith("ARGMAX_PARTIAL") for o in ops) and any(o.startswith("ARGMAX_REDUCE") for o in ops)
    assert per_layer  # (documented order; the counts above are what is asserted)
    if tg is not None:
        names = {t["task_type"] if "task_type" in t else t.get("name") for t in tg.get("all_tasks", [])}
        assert names
    mpk.finalize()


def test_tensor_interleaving_helpers():
    """models/utils.py:42-147 against an element-by-element construction, on the QKV case (uneven chunk sizes) and an inner dim."""
    from mirage.mpk.models.utils import inplace_shuffle_tensors, shuffle_tensors
    g = torch.Generator().manual_seed(3)
    q, k, v = torch.randn(8 * 4, 6, generator=g), torch.randn(4 * 4, 6, generator=g), torch.randn(4 * 4, 6, generator=g)
    out = shuffle_tensors([q, k, v], 4, 0)
    rows = []
    for h in range(4):
        rows += [q[r] for r in range(8 * h, 8 * h + 8)] + [k[r] for r in range(4 * h, 4 * h + 4)] + [v[r] for r in range(4 * h, 4 * h + 4)]
    assert out.shape == (64, 6) and torch.equal(out, torch.stack(rows))
    a, b = torch.arange(12.).reshape(2, 6), 100 + torch.arange(6.).reshape(2, 3)
    assert shuffle_tensors([a, b], 3, -1).tolist() == [[0, 1, 100, 2, 3, 101, 4, 5, 102], [6, 7, 103, 8, 9, 104, 10, 11, 105]]
    tgt = torch.zeros(64, 6, dtype=torch.bfloat16)
    assert inplace_shuffle_tensors([q, k, v], tgt, 4, 0) is None and torch.equal(tgt, out.to(torch.bfloat16))
    for bad, exc in ((lambda: shuffle_tensors([], 2, 0), ValueError), (lambda: shuffle_tensors([q, k], 3, 0), ValueError),
                     (lambda: shuffle_tensors([q, k.double()], 4, 0), TypeError), (lambda: shuffle_tensors([q, k[:, :5]], 4, 0), ValueError),
                     (lambda: shuffle_tensors([q], 4, 2), ValueError), (lambda: shuffle_tensors([q], 0, 0), ValueError)):
        with pytest.raises(exc):
            bad()


def test_wrapper_helpers_of_the_reference(tmp_path, capsys):
    """The small conveniences of the reference's wrapper (mpk.py:102-104, 276-279, 329-341, 369-382, 426-429), host only."""
    import logging
    from mirage.mpk import MPK
    from oracle.qwen3_ref import make_model_weights
    cfg = _cfg()
    md = _metadata(cfg, make_model_weights(cfg, seed=62), "cpu", num_workers=256)
    md.write_to_file(str(tmp_path / "meta.txt"))
    assert (tmp_path / "meta.txt").read_text() == md.info_as_string()
    md.profiling = True
    mpk = MPK(md)
    assert mpk.profiler_tensor.dtype == torch.uint64 and mpk.profiler_tensor.numel() == 3000 * 128
    assert mpk.persistent_kernel.profiler_tensor is mpk.profiler_tensor
    # grids are halved from the last dimension until they fit max_sm_num (108 in the reference's metadata too)
    assert mpk.grid_dim_sanitizer((96, 1, 1)) == (96, 1, 1)
    assert mpk.grid_dim_sanitizer((64, 4, 1)) == (64, 1, 1)
    assert mpk.grid_dim_sanitizer((256, 1, 1)) == (64, 1, 1) and mpk.grid_dim_sanitizer((3, 5, 16)) == (3, 5, 4)
    assert mpk.grid_dim_sanitizer((1, 1, 1)) == (1, 1, 1)
    mpk.print_buffers()
    out = capsys.readouterr().out
    assert out.count("\n") >= 10 and "paged_kv_last_page_len_buffer:" in out and out.startswith("step:")
    seen = []
    lg = logging.getLogger("mpk-test")
    lg.info = lambda msg: seen.append(msg)
    mpk.print_buffers(lg)
    assert len(seen) == 10 and seen[1].startswith("tokens:")
    pk = mpk.persistent_kernel
    del mpk  # the destructor finalizes the kernel ...
    assert pk.__finalized__
    mpk2 = MPK(_metadata(cfg, make_model_weights(cfg, seed=62), "cpu", num_workers=256))
    mpk2.finalize()
    del mpk2  # ... and leaves one the caller finalized alone


def _write_checkpoint(ck, cfg, w, tokenizer=False):
    from safetensors.torch import save_file
    ck.mkdir()
    save_file({k: v.cpu().contiguous() for k, v in _state_dict(w, "cpu").items()}, str(ck / "model.safetensors"))
    (ck / "config.json").write_text(json.dumps({
        "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
        "num_attention_heads": cfg.num_q_heads, "num_key_value_heads": cfg.num_kv_heads, "head_dim": cfg.head_dim,
        "num_hidden_layers": cfg.num_layers, "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_eps, "tie_word_embeddings": False,
        "eos_token_id": 0x7FFFFFF0}))
    if tokenizer:
        # a hand-written word-level tokenizer with the two chat markers as special tokens and a chat template of the Qwen kind
        from tokenizers import Tokenizer, models, pre_tokenizers
        words = ["<unk>", "<|im_start|>", "<|im_end|>", "system", "user", "assistant", "You", "are", "Qwen", ",", "created", "by", "Alibaba", "Cloud", ".",
                 "a", "helpful", "hello", "world", "decode", "me"]
        tok = Tokenizer(models.WordLevel(vocab={wd: i for i, wd in enumerate(words)}, unk_token="<unk>"))
        tok.pre_tokenizer = pre_tokenizers.Whitespace()
        tok.add_special_tokens(["<|im_start|>", "<|im_end|>"])
        tok.save(str(ck / "tokenizer.json"))
        (ck / "tokenizer_config.json").write_text(json.dumps({
            "tokenizer_class": "PreTrainedTokenizerFast", "unk_token": "<unk>", "eos_token": "<|im_end|>",
            "chat_template": "{% for m in messages %}<|im_start|> {{ m['role'] }} {{ m['content'] }} <|im_end|> {% endfor %}"
                             "{% if add_generation_prompt %}<|im_start|> assistant {% endif %}"}))
        return words


def test_checkpoint_with_tokenizer_load_new_request_and_decode(tmp_path):
    """No GPU: a local checkpoint directory WITH tokenizer files -- the string path of load_new_request (chat template, system
    prompt, generation marker: python/mirage/mpk/mpk.py:281-307) and decode().  Skipped if `transformers` cannot load a local
    tokenizer.json offline."""
    from mirage.mpk import MPK
    from oracle.qwen3_ref import make_model_weights
    cfg = _cfg(layers=1, vocab=256)
    w = make_model_weights(cfg, seed=65)
    ck = tmp_path / "qwen3-tiny-tok"
    words = _write_checkpoint(ck, cfg, w, tokenizer=True)
    try:
        from transformers import AutoTokenizer
        AutoTokenizer.from_pretrained(str(ck), local_files_only=True)
    except Exception as e:  # pragma: no cover
        pytest.skip(f"transformers cannot load a local tokenizer here: {e}")
    mpk = MPK(_metadata(cfg, w, "cpu", R=2, T=4, total=2, max_seq=64, PS=16, from_path=str(ck), num_workers=256))
    with pytest.raises(ValueError, match="not built"):
        mpk.load_new_request("hello world")
    mpk.build()
    assert mpk.tokenizer is not None
    ident = {wd: i for i, wd in enumerate(words)}
    mpk.load_new_request("hello world")  # with the chat template
    sys_text = "You are Qwen , created by Alibaba Cloud . You are a helpful assistant ."
    want = [ident[t] for t in ("<|im_start|> system " + sys_text + " <|im_end|> <|im_start|> user hello world <|im_end|> <|im_start|> assistant").split()]
    L = int(mpk.prompt_lengths[0])
    assert L == len(want) and mpk.prompt_lengths.tolist() == [L, L]
    assert mpk.tokens[0, :L].tolist() == want and mpk.tokens[1, :L].tolist() == want and int(mpk.tokens[0, L:].abs().sum()) == 0
    mpk.load_new_request("decode me", use_template=False)
    assert mpk.tokens[0, :int(mpk.prompt_lengths[0])].tolist() == [ident["decode"], ident["me"]]
    assert mpk.decode(torch.tensor([ident["hello"], ident["world"], ident["<|im_end|>"]])) == "hello world"
    mpk.load_new_request([5, 6, 7])  # token ids still work
    assert mpk.tokens[1, :3].tolist() == [5, 6, 7] and mpk.prompt_lengths.tolist() == [3, 3]
    mpk.finalize()


@pytest.mark.gpu
def test_mpk_offline_generation_matches_layer_api_driver_and_oracle(tmp_path):
    from mirage.mpk import MPK
    from oracle.qwen3_ref import make_model_weights, make_prompt
    from test_qwen3_decode import _decoder, _teacher_check
    cfg = _cfg()
    w = make_model_weights(cfg, seed=62)
    R, T, total, max_seq, PS = 3, 8, 5, 40, 16
    prompts = [make_prompt(cfg, n, 700 + i) for i, n in enumerate((5, 11, 8, 3, 17))]
    # the layer-API driver (gang layers), same limits
    dec = _decoder(cfg, w, max_num_batched_tokens=T, max_num_batched_requests=R, max_seq_length=max_seq, page_size=PS, total_requests=total)
    ref_tokens, ref_steps = dec.generate(prompts)
    dec.mpk.finalize()
    # the wrapper + builder, weights handed over as a state dict
    mpk = MPK(_metadata(cfg, w, "cuda", R=R, T=T, total=total, max_seq=max_seq, PS=PS))
    mpk.build()
    mpk.compile()
    _load_prompts(mpk, prompts)
    torch.cuda.synchronize()
    mpk.init_per_request()
    mpk()
    torch.cuda.synchronize()
    toks = mpk.tokens.cpu()
    assert torch.equal(mpk.step.cpu(), ref_steps)
    _teacher_check(cfg, w, prompts, toks, max_seq)
    assert torch.equal(toks, ref_tokens), "the builder's graph and the layer-API driver's graph lower to the same stage program: same tokens"
    assert mpk.persistent_kernel.stats()["aborted"] == 0
    mpk.finalize()
    # a local checkpoint directory: config.json + model.safetensors under the checkpoint's names
    ck = tmp_path / "qwen3-tiny"
    _write_checkpoint(ck, cfg, w)
    mpk2 = MPK(_metadata(cfg, w, "cuda", R=R, T=T, total=total, max_seq=max_seq, PS=PS, from_path=str(ck)))
    mpk2.build()
    assert mpk2.tokenizer is None  # no tokenizer files in the directory: token ids in, token ids out
    mpk2.compile()
    _load_prompts(mpk2, prompts)
    torch.cuda.synchronize()
    mpk2.init_per_request()
    mpk2()
    torch.cuda.synchronize()
    assert torch.equal(mpk2.tokens.cpu(), ref_tokens), "checkpoint-loaded weights must give the state-dict run's tokens"
    mpk2.finalize()


@pytest.mark.gpu
def test_mpk_run_same_prompt_in_every_slot():
    """MPK.run(prompt): the same prompt in every request slot, rows identical (the reference driver's self-check,
    demo/qwen3/demo.py:1281-1301)."""
    from mirage.mpk import MPK
    from oracle.qwen3_ref import make_model_weights, make_prompt
    cfg = _cfg()
    w = make_model_weights(cfg, seed=63)
    md = _metadata(cfg, w, "cuda", R=4, T=32, total=4, max_seq=36, PS=16)
    mpk = MPK(md)
    mpk.build()
    out = mpk.run(make_prompt(cfg, 8, 9))
    assert len(out) == 4 and all(torch.equal(o, out[0]) for o in out)
    assert out[0].numel() == 36
    mpk.finalize()


@pytest.mark.gpu
def test_mpk_online_notoken_returns_normalised_hidden_state():
    from mirage.mpk import MPK
    from oracle.qwen3_ref import KVCache, Qwen3Oracle, make_model_weights, make_prompt
    cfg = _cfg()
    w = make_model_weights(cfg, seed=64)
    P, max_seq, PS = 7, 32, 16
    prompt = make_prompt(cfg, P, 3)
    mpk = MPK(_metadata(cfg, w, "cuda", mode="online_notoken", R=1, T=8, total=1, max_seq=max_seq, PS=PS, with_lm_head=False))
    mpk.build()
    mpk.compile()
    # the caller describes the batch: one request, P new tokens at positions 0..P-1, one page
    mpk.input_tokens[:P, 0].copy_(prompt.cuda())
    mpk.qo_indptr_buffer.copy_(torch.tensor([0, P], dtype=torch.int32))
    mpk.paged_kv_indptr_buffer.copy_(torch.tensor([0, 1], dtype=torch.int32))
    mpk.paged_kv_indices_buffer.zero_()
    mpk.paged_kv_last_page_len_buffer.copy_(torch.tensor([P], dtype=torch.int32))
    torch.cuda.synchronize()
    hidden = mpk()
    torch.cuda.synchronize()
    assert hidden is not None and tuple(hidden.shape) == (8, cfg.hidden_size)
    # Two legitimate summation orders (fp32 and exact sums at the same rounding points) already differ in about half
    # of the elements after two layers and a norm; the GPU (a third order) must sit as close to the exact-sum oracle
    # as the fp32 oracle does, and point the same way.
    o32, o64 = Qwen3Oracle(cfg, w, "kernel"), Qwen3Oracle(cfg, w, "kernel", acc=torch.float64)
    o32.forward(prompt, KVCache(cfg, max_seq), 0)
    o64.forward(prompt, KVCache(cfg, max_seq), 0)
    h, h32, h64 = hidden[:P].cpu().float(), o32.last_hidden.float(), o64.last_hidden.float()
    drift = float((h32 - h64).abs().max())
    err = float((h - h64).abs().max())
    assert err <= 1.5 * drift + 2.0 ** -7, f"GPU is {err} from the exact-sum oracle; the fp32-sum oracle is {drift} from it"
    cos = torch.nn.functional.cosine_similarity(h.flatten(), h64.flatten(), dim=0)
    assert float(cos) > 0.9999
    mpk.finalize()
