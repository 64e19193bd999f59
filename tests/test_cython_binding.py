"""The compiled Cython binding (mirage/_cython/core.pyx, built by build.py) against the ctypes one: the same C ABI, the same
results.  Counterpart of the reference's python/mirage/_cython/core.pyx for this library."""
import pytest
import torch

import mirage as mi
from helpers import make_meta
from mirage import _capi


def _mpk(binding, B=4, R=2, max_seq=64):
    meta = make_meta(R, max_seq, B, R, 8, device="cpu")
    return mi.PersistentKernel(mode="offline", world_size=1, mpi_rank=0, num_workers=256, num_local_schedulers=0, num_remote_schedulers=0,
                               max_seq_length=max_seq, max_num_batched_requests=R, max_num_batched_tokens=B, max_num_pages=8, page_size=16,
                               meta_tensors=meta, profiler_tensor=None, trace_name=None, spec_decode_config=None, use_cutlass_kernel=False,
                               eos_token_id=2, binding=binding)


def _record_small_graph(mpk):
    z = lambda name, *shape, dtype=torch.bfloat16: mpk.attach_input(torch.zeros(*shape, dtype=dtype), name)
    ids = z("ids", 4, 1, dtype=torch.int64)
    emb, x = z("embed", 64, 1024), mpk.new_tensor(dims=(4, 1024), dtype=mi.bfloat16, name="x", io_category="cuda_tensor")
    mpk.embed_layer(input=ids, weight=emb, output=x, grid_dim=(1, 1, 1), block_dim=(128, 1, 1), input_source=1)
    nw, n = z("nw", 1024), mpk.new_tensor(dims=(4, 1024), dtype=mi.bfloat16, name="n", io_category="cuda_tensor")
    mpk.rmsnorm_layer(input=x, weight=nw, output=n, grid_dim=(4, 1, 1), block_dim=(128, 1, 1))
    q, k, v = z("q", 1024, 1024), z("k", 256, 1024), z("v", 256, 1024)
    qkv = mpk.shuffle_tensors([q, k, v], 0, 2, "qkv")
    y = mpk.new_tensor(dims=(4, 1536), dtype=mi.bfloat16, name="y", io_category="cuda_tensor")
    mpk.linear_layer(input=n, weight=qkv, output=y, grid_dim=(24, 1, 1), block_dim=(128, 1, 1))
    return y


def test_module_is_built_and_names_the_same_library():
    from mirage._cython import core
    lib = _capi.load()
    assert core.version() == lib.mk_version().decode()
    assert core.CyGraph.binding == "cython" and _capi.Graph.binding == "ctypes"
    with pytest.raises(ValueError, match="unknown binding"):
        _capi.make_graph({}, "pybind")


def test_same_program_and_task_graph_through_both_bindings():
    out = {}
    for binding in ("ctypes", "cython"):
        mpk = _mpk(binding)
        assert mpk._g.binding == binding and mpk._handle.value == mpk._g.handle != 0
        y = _record_small_graph(mpk)
        assert (y.num_dims, y.dim(1)) == (2, 1536)
        out[binding] = (mpk.describe_program(), mpk.kn_graph.generate_task_graph(1, 0)["json_file"], mpk.stats())
        mpk.finalize()
    assert out["ctypes"][0] == out["cython"][0] and "LINEAR+norm" in out["cython"][0]
    assert out["ctypes"][1] == out["cython"][1] and '"all_tasks"' in out["cython"][1]
    assert out["ctypes"][2] == out["cython"][2]


def test_errors_carry_the_library_message():
    for binding in ("ctypes", "cython"):
        mpk = _mpk(binding)
        with pytest.raises(_capi.MkError, match="Unsupported task name"):
            mpk._g.add_task("no_such_task", (1, 1, 1), (128, 1, 1), [], [], [], [])
        with pytest.raises(_capi.MkError, match="without a device"):
            mpk._g.compile()
        with pytest.raises(KeyError, match="no field"):
            _capi.make_graph({"not_a_field": 1}, binding)
        with pytest.raises(_capi.MkError):  # a configuration the library rejects
            _capi.make_graph({"max_seq_length": 0}, binding)
        mpk.finalize()
    with pytest.raises(ValueError, match="three"):
        _mpk("cython")._g.add_task("linear", (1, 1), (128, 1, 1), [], [], [], [])


@pytest.mark.gpu
def test_generation_is_identical_through_the_cython_binding(monkeypatch):
    from oracle.qwen3_ref import make_model_weights, make_prompt
    from test_qwen3_decode import _decoder, _small_cfg
    cfg = _small_cfg()
    w = make_model_weights(cfg, seed=7)
    prompts = [make_prompt(cfg, 9, 1), make_prompt(cfg, 5, 2)]
    toks = {}
    for binding in ("ctypes", "cython"):
        monkeypatch.setenv("FLEET_MK_BINDING", binding)
        dec = _decoder(cfg, w, max_num_batched_tokens=8, max_num_batched_requests=2, max_seq_length=40, page_size=16)
        assert dec.mpk._g.binding == binding
        toks[binding] = dec.generate(prompts)
        st = dec.mpk.stats()
        prof = dec.mpk.stage_profile(0, raw=True)
        assert st["iterations"] > 30 and len(prof) == st["num_stages"] + 1
        # bounded launches, the host-side wait and the profiler tensor through the same binding
        dec.load_prompts(prompts)
        dec.mpk.profiler_tensor = torch.zeros(1 << 14, dtype=torch.uint64, device="cuda")
        dec.mpk.enqueue_steps(5)
        assert dec.mpk.wait() is False
        assert dec.mpk.run_steps(1 << 20) is True
        assert torch.equal(dec.meta["tokens"].cpu(), toks[binding][0])
        assert int((dec.mpk.profiler_tensor.cpu().view(torch.int64) != 0).sum()) > 100
        dec.mpk.finalize()
    assert torch.equal(toks["ctypes"][0], toks["cython"][0]) and torch.equal(toks["ctypes"][1], toks["cython"][1])
