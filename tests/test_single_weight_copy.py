"""One resident copy of the weights (no counterpart in the reference, whose drivers keep the row-major QKV and gate/up
weights AND an interleaved copy of them, src/kernel/runtime.cc:904-943): a graph built with single_weight_copy keeps every
linear weight once, in matrix-core tile order; the attached row-major tensors can be freed after compile(), and iterations
of one and two tokens run the matrix-core forms.  Checked: the same parity bars as the two-copy default (stage by stage at
full width, end to end against the oracle), that the kernel really never reads the released tensors (they are overwritten
with NaN and freed), and the byte accounting."""
import gc

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_new", [1, 2, 8])
def test_full_width_layer_stagewise_from_the_tile_copy_only(n_new):
    from helpers import check_layer_stages
    from oracle.qwen3_ref import Qwen3Config
    from test_qwen3_layer import _run_layer
    cfg = Qwen3Config(num_layers=1)
    res = _run_layer(cfg, 130, n_new, "fleet", seed=60 + n_new, batch_tokens=8, single_weight_copy=True)
    check_layer_stages(res, cfg, 130, n_new)
    assert res["stats"]["row_major_weight_bytes"] == 0
    assert res["stats"]["packed_weight_bytes"] == 2 * (6144 * 4096 + 4096 * 4096 + 24576 * 4096 + 4096 * 12288)
    assert "NORM" in res["program"]


def test_generation_after_the_row_major_weights_are_gone():
    """Continuous batching with 1..8-token iterations on a small model: tokens agree with the oracle, the released
    tensors are poisoned and freed, and a second generation reproduces the first bit for bit."""
    from mirage import _capi
    from oracle.qwen3_ref import make_model_weights, make_prompt
    from test_qwen3_decode import _decoder, _small_cfg, _teacher_check
    cfg = _small_cfg()
    w = make_model_weights(cfg, seed=23)
    R, B, total, max_seq = 3, 8, 5, 40
    prompts = [make_prompt(cfg, n, 900 + i) for i, n in enumerate((5, 11, 8, 3, 17))]
    ref = _decoder(cfg, w, max_num_batched_tokens=B, max_num_batched_requests=R, max_seq_length=max_seq, page_size=16, total_requests=total)
    st0 = ref.mpk.stats()
    linear_bytes = st0["weight_bytes"]
    assert st0["row_major_weight_bytes"] == linear_bytes == st0["packed_weight_bytes"]  # the default: both copies
    assert ref.mpk.release_row_major_weights() == []
    ref.mpk.finalize()
    del ref
    torch.cuda.synchronize()
    dec = _decoder(cfg, w, max_num_batched_tokens=B, max_num_batched_requests=R, max_seq_length=max_seq, page_size=16, total_requests=total,
                   single_weight_copy=True)
    st = dec.mpk.stats()
    assert st["row_major_weight_bytes"] == 0 and st["packed_weight_bytes"] == linear_bytes
    toks1, steps1 = dec.generate(prompts)
    _teacher_check(cfg, w, prompts, toks1, max_seq)
    released = dec.mpk.release_row_major_weights()
    per_layer = {"q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"}
    assert sorted(released) == sorted([f"layer_{i}_{k}" for i in range(cfg.num_layers) for k in per_layer] + ["lm_head"])
    # poison, then free: the decoder's weight dict holds the only other references
    before = torch.cuda.memory_allocated()
    for lw in dec.w["layers"]:
        for k in per_layer:
            lw[k].fill_(float("nan"))
            del lw[k]
    dec.w["lm_head"].fill_(float("nan"))
    del dec.w["lm_head"]
    torch.cuda.synchronize()
    freed = before - torch.cuda.memory_allocated()
    assert freed >= 0.95 * linear_bytes, f"freed {freed} of {linear_bytes} bytes"
    toks2, steps2 = dec.generate(prompts)
    assert torch.equal(toks1, toks2) and torch.equal(steps1, steps2)
    with pytest.raises(_capi.MkError, match="only the tile copies"):
        dec.mpk.repack_weights()
    assert dec.mpk.stats()["aborted"] == 0
    dec.mpk.finalize()


def test_tied_head_and_unpackable_weights():
    """A weight that another stage reads row-major (the embedding table used as LM head) stays; a linear whose reduction
    length cannot be tiled makes compile() refuse the mode."""
    import mirage as mi
    from helpers import make_meta, make_mpk
    from mirage import _capi
    B, H, V = 4, 1024, 512
    meta = make_meta(B, 64, B, B, B)

    def build(k_head, flag=True):
        mpk = mi.PersistentKernel(mode="onepass", world_size=1, mpi_rank=0, num_workers=256, num_local_schedulers=0, num_remote_schedulers=0, max_seq_length=64,
                                  max_num_batched_requests=B, max_num_batched_tokens=B, max_num_pages=B, page_size=64, meta_tensors=meta, profiler_tensor=None,
                                  trace_name=None, spec_decode_config=None, use_cutlass_kernel=False, single_weight_copy=flag)
        table = torch.randn(V, H, device="cuda").to(torch.bfloat16)
        ids = mpk.attach_input(meta["input_tokens"], "ids")
        tw = mpk.attach_input(table, "embed")
        x, y, z = mpk.new_tensor((B, H), name="x"), mpk.new_tensor((B, k_head), name="y"), mpk.new_tensor((B, V), name="z")
        mpk.embed_layer(input=ids, weight=tw, output=x, grid_dim=(1, 1, 1), block_dim=(128, 1, 1), input_source=1)
        w1 = mpk.attach_input(torch.randn(k_head, H, device="cuda").to(torch.bfloat16), "w1")
        mpk.linear_layer(input=x, weight=w1, output=y, grid_dim=(k_head // 8, 1, 1), block_dim=(128, 1, 1))
        head = mpk.attach_input(table[:, :k_head].contiguous() if k_head != H else table, "tied_head")
        mpk.linear_layer(input=y, weight=head, output=z, grid_dim=(V // 64, 1, 1), block_dim=(128, 1, 1))
        return mpk

    mpk = build(H)
    mpk.compile()
    assert mpk.release_row_major_weights() == ["w1"]  # "tied_head" is the embedding table's memory
    assert mpk.stats()["row_major_weight_bytes"] == V * H * 2
    mpk.finalize()
    mpk = build(992)  # 992 = 31 * 32: the second linear's reduction length is not a multiple of 64
    with pytest.raises(_capi.MkError, match="cannot be laid out in matrix-core tiles"):
        mpk.compile()
    mpk.finalize()


def test_checkpoint_loaded_model_holds_its_linears_once(tmp_path):
    """MPK + Qwen3Builder from a local safetensors directory: with single_weight_copy the row-major linears the loader put
    on the GPU are dropped at compile(), so the process holds the model once (tile copies) instead of twice; the tokens pass
    the oracle check."""
    from mirage.mpk import MPK
    from oracle.qwen3_ref import make_model_weights, make_prompt
    from test_mpk_builder import _cfg, _load_prompts, _metadata, _write_checkpoint
    from test_qwen3_decode import _teacher_check
    cfg = _cfg()
    w = make_model_weights(cfg, seed=66)
    ck = tmp_path / "qwen3-tiny"
    _write_checkpoint(ck, cfg, w)
    R, T, total, max_seq, PS = 3, 8, 5, 40, 16
    prompts = [make_prompt(cfg, n, 700 + i) for i, n in enumerate((5, 11, 8, 3, 17))]
    held = {}
    for single in (False, True):
        gc.collect()  # (what earlier tests left in reference cycles must not be freed inside the measured window)
        torch.cuda.synchronize()
        base = torch.cuda.memory_allocated()
        md = _metadata(cfg, w, "cuda", R=R, T=T, total=total, max_seq=max_seq, PS=PS, from_path=str(ck))
        md.single_weight_copy = single
        mpk = MPK(md)
        mpk.build()
        mpk.compile()
        torch.cuda.synchronize()
        held[single] = torch.cuda.memory_allocated() - base  # torch-side memory: the loader's tensors, caches, meta tensors
        st = mpk.persistent_kernel.stats()
        linear = st["weight_bytes"]
        assert st["packed_weight_bytes"] == linear and st["row_major_weight_bytes"] == (0 if single else linear)
        _load_prompts(mpk, prompts)
        torch.cuda.synchronize()
        mpk.init_per_request()
        mpk()
        torch.cuda.synchronize()
        _teacher_check(cfg, w, prompts, mpk.tokens.cpu(), max_seq)
        mpk.finalize()
        del mpk, md
    assert held[False] - held[True] >= 0.95 * linear, f"torch holds {held[False]} bytes with both copies and {held[True]} with one; the linears are {linear} bytes"
