"""Grid helpers of the model builders (reference: python/mirage/mpk/models/utils.py:3-42).  The weight-interleaving
helpers of that file have no counterpart: interleaved weights are views here (PersistentKernel.shuffle_tensors)."""


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
