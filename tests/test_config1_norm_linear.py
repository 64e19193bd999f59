"""Headline configuration 1: RMSNorm(4096) -> linear 4096x4096, BS=1 bf16, as a two-task graph through the C ABI.

Closest reference checks (CUDA-only, formula only): tests/runtime_python/test_norm_linear.py:13-19."""
import pytest
import torch

from helpers import bf16_ulp_diff, make_meta, make_mpk

pytestmark = pytest.mark.gpu


def _inputs(H, N, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(1, H, generator=g).to(torch.bfloat16)
    nw = (1.0 + 0.02 * torch.randn(H, generator=g)).to(torch.bfloat16)
    W = (0.02 * torch.randn(N, H, generator=g)).to(torch.bfloat16)
    return x, nw, W


@pytest.mark.parametrize("gang", [False, True])
@pytest.mark.parametrize("H,N", [(4096, 4096), (1024, 3000), (12288, 512)])
def test_norm_linear_bs1(gang, H, N):
    import mirage as mi
    from oracle.qwen3_ref import linear_k, rmsnorm_k
    if gang and (N % 8 or (N // 8) % 64):
        pytest.skip("gang layers need N divisible by 8*tile_n")
    x, nw, W = _inputs(H, N)
    meta = make_meta(1, 64, 1, 1, 1)
    mpk = make_mpk(meta, 64, 1, 1, 1, 64, mode="onepass")
    xd, nwd, Wd = x.cuda(), nw.cuda(), W.cuda()
    tx = mpk.attach_input(xd, "x")
    tnw = mpk.attach_input(nwd, "norm_w")
    tW = mpk.attach_input(Wd, "W")
    tn = mpk.new_tensor((1, H), dtype=mi.bfloat16, name="norm_out")
    ty = mpk.new_tensor((1, N), dtype=mi.bfloat16, name="y")
    if gang:
        mpk.gang_rmsnorm_layer(input=tx, weight=tnw, output=tn)
        mpk.gang_linear_layer(input=tn, weight=tW, output=ty, tile_n=64, output_stride=N)
    else:
        mpk.rmsnorm_layer(input=tx, weight=tnw, output=tn, grid_dim=(1, 1, 1), block_dim=(128, 1, 1))
        mpk.linear_layer(input=tn, weight=tW, output=ty, grid_dim=(N // 8 if N % 8 == 0 else 1, 1, 1), block_dim=(128, 1, 1))
    mpk.compile()
    mpk.run_once([0], [0])
    y = ty.to_torch().cpu()
    n_gpu = tn.to_torch().cpu()
    n_ref = rmsnorm_k(x, nw)
    y_ref = linear_k(n_ref, W)
    # the fused norm output must be bit-exact up to rsqrt rounding: allow 1 bf16 ulp
    ulp_n, _ = bf16_ulp_diff(n_gpu, n_ref)
    assert ulp_n <= 1.0, f"norm differs by {ulp_n} bf16 ulp"
    # fp32 accumulation order differs from torch's matmul: allow 1 bf16 ulp of the row scale + small abs
    torch.testing.assert_close(y.float(), y_ref.float(), atol=2e-2, rtol=1e-2)  # north-star tolerance
    d = (y.float() - y_ref.float()).abs()
    assert float(d.max()) <= 0.016, f"max abs diff {float(d.max())}"
    assert float((d > 0).float().mean()) < 0.05, "more than 5% of outputs differ from the fp32-accumulate oracle"
    st = mpk.stats()
    assert st["num_xcds"] == 8 and st["aborted"] == 0
    mpk.finalize()


@pytest.mark.parametrize("M", [2, 5, 16, 17, 33, 64])
@pytest.mark.parametrize("H,N,res", [(4096, 4096, True), (1024, 3008, False), (12288, 512, True)])
def test_norm_linear_multi_token(M, H, N, res):
    """Multi-token rows take the MFMA path (norm as its own stage, linear with optional residual)."""
    import mirage as mi
    from oracle.qwen3_ref import linear_k, rmsnorm_k
    g = torch.Generator().manual_seed(M * 7 + N)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    nw = (1.0 + 0.02 * torch.randn(H, generator=g)).to(torch.bfloat16)
    W = (0.02 * torch.randn(N, H, generator=g)).to(torch.bfloat16)
    r = torch.randn(M, N, generator=g).to(torch.bfloat16)
    B = 64
    meta = make_meta(1, 64, B, B, B)
    mpk = make_mpk(meta, 64, B, B, B, 64, mode="onepass")
    pad = lambda t: torch.cat([t, torch.zeros(B - t.shape[0], t.shape[1], dtype=t.dtype)]).cuda()
    xd, nwd, Wd, rd = pad(x), nw.cuda(), W.cuda(), pad(r)
    tx, tnw, tW, tr = mpk.attach_input(xd, "x"), mpk.attach_input(nwd, "norm_w"), mpk.attach_input(Wd, "W"), mpk.attach_input(rd, "res")
    tn = mpk.new_tensor((B, H), dtype=mi.bfloat16, name="norm_out")
    ty = mpk.new_tensor((B, N), dtype=mi.bfloat16, name="y")
    mpk.rmsnorm_layer(input=tx, weight=tnw, output=tn, grid_dim=(B, 1, 1), block_dim=(128, 1, 1))
    if res:
        mpk.linear_with_residual_layer(input=tn, weight=tW, residual=tr, output=ty, grid_dim=(N // 64, 1, 1), block_dim=(256, 1, 1))
    else:
        mpk.linear_layer(input=tn, weight=tW, output=ty, grid_dim=(N // 64, 1, 1), block_dim=(128, 1, 1))
    mpk.compile()
    mpk.run_once(list(range(M)), [0] * M)   # M requests with one token each
    y = ty.to_torch().cpu()
    n_gpu = tn.to_torch().cpu()
    n_ref = rmsnorm_k(x, nw)
    ulp_n, _ = bf16_ulp_diff(n_gpu[:M], n_ref)
    assert ulp_n <= 1.0
    y_ref = linear_k(n_gpu[:M], W, res=r if res else None)   # oracle fed with the GPU's own normalised rows
    frac = float((y[:M].float() != y_ref.float()).float().mean())
    ulp, mabs = bf16_ulp_diff(y[:M], y_ref, floor=1.0 / 16)
    assert ulp <= 1.0 and frac < 0.02, f"{frac:.4f} of outputs differ, max {ulp} ulp ({mabs})"
    assert float(y[M:].abs().sum()) == 0.0, "rows beyond the batch must not be written"
    assert mpk.stats()["aborted"] == 0
    mpk.finalize()


@pytest.mark.parametrize("M", [16, 50])
def test_linear_wide_range_sweeps(M):
    """A stage with many tiles per workgroup (LM-head-like: 70000 rows, not a multiple of 16) on the matrix-core path:
    each workgroup works its tile range off in several sweeps, the last one ragged."""
    import mirage as mi
    from oracle.qwen3_ref import linear_k
    H, N = 1024, 70000
    g = torch.Generator().manual_seed(M)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    W = (0.02 * torch.randn(N, H, generator=g)).to(torch.bfloat16)
    B = 64
    meta = make_meta(1, 64, B, B, B)
    mpk = make_mpk(meta, 64, B, B, B, 64, mode="onepass")
    xd = torch.cat([x, torch.zeros(B - M, H, dtype=x.dtype)]).cuda()
    tx, tW = mpk.attach_input(xd, "x"), mpk.attach_input(W.cuda(), "W")
    ty = mpk.new_tensor((B, N), dtype=mi.bfloat16, name="y")
    mpk.linear_layer(input=tx, weight=tW, output=ty, grid_dim=(64, 1, 1), block_dim=(128, 1, 1))
    mpk.compile()
    mpk.run_once(list(range(M)), [0] * M)
    y = ty.to_torch().cpu()
    y_ref = linear_k(x, W)
    frac = float((y[:M].float() != y_ref.float()).float().mean())
    ulp, mabs = bf16_ulp_diff(y[:M], y_ref, floor=1.0 / 16)
    assert ulp <= 1.0 and frac < 0.02, f"{frac:.4f} of outputs differ, max {ulp} ulp ({mabs})"
    assert float(y[M:].abs().sum()) == 0.0, "rows beyond the batch must not be written"
    assert mpk.stats()["aborted"] == 0
    mpk.finalize()


@pytest.mark.parametrize("M", [16, 64])
def test_linear_silu_split_k(M):
    """A SwiGLU linear with few tiles per workgroup (2048 interleaved [gate ; up] rows, K = 4096) on the matrix-core
    path: the reduction is split over workgroups, the gate and up partial sums are combined before the activation."""
    import mirage as mi
    from oracle.qwen3_ref import linear_silu_k
    H, I, TN = 4096, 1024, 128  # a physically interleaved weight uses the reference layout [gate128 ; up128]
    g = torch.Generator().manual_seed(100 + M)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    Wg = (0.02 * torch.randn(I, H, generator=g)).to(torch.bfloat16)
    Wu = (0.02 * torch.randn(I, H, generator=g)).to(torch.bfloat16)
    W = torch.cat([torch.cat([Wg[i:i + TN], Wu[i:i + TN]]) for i in range(0, I, TN)])  # [gate ; up] groups of TN rows
    B = 64
    meta = make_meta(1, 64, B, B, B)
    mpk = make_mpk(meta, 64, B, B, B, 64, mode="onepass")
    xd = torch.cat([x, torch.zeros(B - M, H, dtype=x.dtype)]).cuda()
    tx, tW = mpk.attach_input(xd, "x"), mpk.attach_input(W.cuda(), "W")
    ty = mpk.new_tensor((B, I), dtype=mi.bfloat16, name="y")
    mpk.linear_silu_layer(input=tx, weight=tW, output=ty, output_stride=I, tile_n=64)
    mpk.compile()
    mpk.run_once(list(range(M)), [0] * M)
    y = ty.to_torch().cpu()
    y_ref = linear_silu_k(x, Wg, Wu)
    frac = float((y[:M].float() != y_ref.float()).float().mean())
    ulp, mabs = bf16_ulp_diff(y[:M], y_ref, floor=1.0 / 16)
    assert ulp <= 1.0 and frac < 0.02, f"{frac:.4f} of outputs differ, max {ulp} ulp ({mabs})"
    assert mpk.stats()["aborted"] == 0
    mpk.finalize()
