"""Every linear-type layer builder of the reference API must lower to the same mathematics: out = x W^T (+ residual).

The reference driver switches between these builders with environment variables (demo/qwen3/demo.py:805-885,1025-1113:
USE_GANG_KSPLIT, USE_GANG_SPLITK, USE_GANG_M_SPLIT, USE_GANG_N_TILE, the split-K atomic path of its non-gang mode); each
has its own operand order (python/mirage/mpk/persistent_kernel.py:1437-1560,1618-1850,1920-1990).  Here each builder is
called with that operand order on distinct tensors (so a swapped operand changes the result or fails validation) and
compared with the fp32-accumulate oracle at one, eight and sixty-four tokens (dot-product, few-token and matrix-core
forms of the stage)."""
import pytest
import torch

from helpers import bf16_ulp_diff, make_meta, make_mpk

pytestmark = pytest.mark.gpu

H, N = 4096, 4096

BUILDERS = ["linear", "linear_with_residual", "splitk_linear", "splitk_linear_res_atomic", "gang_linear", "gang_linear_n_tiling",
            "gang_linear_with_residual", "gang_linear_with_residual_n_tiling", "gang_linear_msplit", "gang_linear_with_residual_msplit",
            "gang_splitk_linear_with_residual", "gang_ksplit_linear_with_residual"]


def _build(mpk, name, t, B):
    x, W, r, ws, dc, y = t["x"], t["W"], t["r"], t["ws"], t["dc"], t["y"]
    m_tiles = 2 if B % 2 == 0 else 1
    if name == "linear":
        mpk.linear_layer(input=x, weight=W, output=y, grid_dim=(N // 64, 1, 1), block_dim=(128, 1, 1))
    elif name == "linear_with_residual":
        mpk.linear_with_residual_layer(input=x, weight=W, residual=r, output=y, grid_dim=(N // 64, 1, 1), block_dim=(256, 1, 1))
    elif name == "splitk_linear":
        mpk.splitk_linear_layer(input=x, weight=W, output=y, grid_dim=(N // 64, 4, 1), block_dim=(256, 1, 1))
    elif name == "splitk_linear_res_atomic":
        mpk.splitk_linear_res_atomic_layer(input=x, weight=W, residual=r, workspace=ws, done_counter=dc, output=y, k_splits=4,
                                           grid_dim=(N // 64, 4, 1), block_dim=(256, 1, 1))
    elif name == "gang_linear":
        mpk.gang_linear_layer(input=x, weight=W, output=y, tile_n=64, output_stride=N, m_tiles=1)
    elif name == "gang_linear_n_tiling":
        mpk.gang_linear_n_tiling_layer(input=x, weight=W, output=y, tile_n=64, output_stride=N, m_tiles=1, wgn=0)
    elif name == "gang_linear_with_residual":
        mpk.gang_linear_with_residual_layer(input=x, weight=W, residual=r, output=y, tile_n=64, output_stride=N, m_tiles=1)
    elif name == "gang_linear_with_residual_n_tiling":
        mpk.gang_linear_with_residual_n_tiling_layer(input=x, weight=W, residual=r, output=y, tile_n=64, output_stride=N, m_tiles=1, wgn=0)
    elif name == "gang_linear_msplit":
        mpk.gang_linear_msplit_layer(input=x, weight=W, output=y, tile_n=64, output_stride=N, m_tiles=m_tiles)
    elif name == "gang_linear_with_residual_msplit":
        mpk.gang_linear_with_residual_msplit_layer(input=x, weight=W, residual=r, output=y, tile_n=64, output_stride=N, m_tiles=m_tiles)
    elif name == "gang_splitk_linear_with_residual":
        mpk.gang_splitk_linear_with_residual_layer(input=x, weight=W, residual=r, workspace=ws, output=y, tile_n=64, output_stride=N, k_splits=4)
    elif name == "gang_ksplit_linear_with_residual":
        mpk.gang_ksplit_linear_with_residual_layer(input=x, weight=W, residual=r, workspace=ws, output=y, tile_n=64, output_stride=N, k_splits=8)
    else:
        raise AssertionError(name)
    return "residual" in name or "res_" in name


@pytest.mark.parametrize("M,B", [(1, 1), (8, 8), (64, 64)])
@pytest.mark.parametrize("name", BUILDERS)
def test_linear_builder_matches_oracle(name, M, B):
    import mirage as mi
    from oracle.qwen3_ref import linear_k
    g = torch.Generator().manual_seed(BUILDERS.index(name) * 97 + M)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    W = (0.02 * torch.randn(N, H, generator=g)).to(torch.bfloat16)
    r = torch.randn(M, N, generator=g).to(torch.bfloat16)
    meta = make_meta(1, 64, B, B, B)
    mpk = make_mpk(meta, 64, B, B, B, 64, mode="onepass")
    dev = [x.cuda(), W.cuda(), r.cuda(), torch.zeros(B, N, dtype=torch.float32, device="cuda"), torch.zeros(N // 64, 1, dtype=torch.int32, device="cuda")]
    t = {"x": mpk.attach_input(dev[0], "x"), "W": mpk.attach_input(dev[1], "W"), "r": mpk.attach_input(dev[2], "res"),
         "ws": mpk.attach_input(dev[3], "splitk_workspace"), "dc": mpk.attach_input(dev[4], "splitk_done_counter"),
         "y": mpk.new_tensor((B, N), dtype=mi.bfloat16, name="y")}
    has_res = _build(mpk, name, t, B)
    mpk.compile()
    mpk.run_once(list(range(M)), [0] * M)
    y = t["y"].to_torch().cpu()
    y_ref = linear_k(x, W, res=r if has_res else None)
    frac = float((y.float() != y_ref.float()).float().mean())
    ulp, mabs = bf16_ulp_diff(y, y_ref, floor=1.0 / 16)
    assert ulp <= 1.0 and frac < 0.02, f"{name}: {frac:.4f} of outputs differ, max {ulp} ulp ({mabs})"
    assert mpk.stats()["aborted"] == 0
    mpk.finalize()
