"""Helpers of the model builders (reference: python/mirage/mpk/models/utils.py).  The builders here never copy weights
to interleave them (PersistentKernel.shuffle_tensors records a view that the kernel resolves); the two tensor-level
interleaving helpers are kept for callers that prepare fused weights themselves."""
import torch


def grid_for_rmsnorm_linear_layer(size: int) -> int:
    """Blocks the reference gives a norm+linear task over `size` output rows: 96 or 64 when they divide it, size/256 for
    very wide outputs, else the largest small divisor."""
    if size / 96 > 400:
        assert size % 256 == 0, f"FATAL: Linear layer size not support, it's {size}."
        return size // 256
    for d in (96, 64, 48, 32, 24, 18, 16, 12, 9, 8, 6, 4, 3, 2, 1):
        if size % d == 0:
            return d
    return 1


def max_factor_leq_n(m: int, n: int) -> int:
    """Largest factor of m that is <= n."""
    best, i = 1, 1
    while i * i <= m:
        if m % i == 0:
            if i <= n:
                best = max(best, i)
            if m // i <= n:
                best = max(best, m // i)
        i += 1
    return best


def shuffle_tensors(tensors, split: int, dim: int) -> torch.Tensor:
    """A new tensor in which the `split` equal chunks of every input along `dim` alternate in input order: [Q, K, V] with
    split = number of kv heads gives [Q_0, K_0, V_0, Q_1, K_1, V_1, ...] (models/utils.py:42-118)."""
    if not tensors:
        raise ValueError("tensors must be a non-empty list")
    first = tensors[0]
    nd = first.ndim
    if not -nd <= dim < nd:
        raise ValueError(f"dim out of range for {nd}-D tensor: {dim}")
    dim %= nd
    if split <= 0:
        raise ValueError("split must be a positive integer")
    for i, t in enumerate(tensors):
        if t.dtype != first.dtype or t.device != first.device:
            raise TypeError(f"tensor {i} is {t.dtype} on {t.device}, the first one {first.dtype} on {first.device}")
        if t.ndim != nd or any(t.shape[d] != first.shape[d] for d in range(nd) if d != dim):
            raise ValueError(f"tensor {i} has shape {tuple(t.shape)}: all dimensions but {dim} must match {tuple(first.shape)}")
        if t.shape[dim] % split:
            raise ValueError(f"tensor {i} has {t.shape[dim]} entries along dim {dim}, not a multiple of split={split}")
    chunks = [t.chunk(split, dim=dim) for t in tensors]
    return torch.cat([c[i] for i in range(split) for c in chunks], dim=dim)


def inplace_shuffle_tensors(tensors, target_tensor: torch.Tensor, split: int, dim: int) -> None:
    """The same interleaving written into `target_tensor` (its device and dtype; models/utils.py:120-147)."""
    if not tensors:
        raise ValueError("tensors must be a non-empty list")
    out = shuffle_tensors([t.to(device=target_tensor.device, dtype=target_tensor.dtype) for t in tensors], split, dim)
    assert out.shape == target_tensor.shape, f"interleaved shape {tuple(out.shape)} does not match the target's {tuple(target_tensor.shape)}"
    target_tensor.copy_(out)
