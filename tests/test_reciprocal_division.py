"""The index arithmetic of the broadcasting kernels divides by the extents of the merged axis groups through a
multiplication: n / d = (n * magic) >> shift with shift = 31 + ceil(log2 d) and magic = floor(2^shift / d) + 1, which
has to be exact for every n below 2^31 (the kernels take this path only for tensors of fewer than 2^31 elements).
Checked here in exact integer arithmetic: every divisor up to 4096 and a spread of larger ones, against n at the
places where a rounded reciprocal goes wrong first (multiples of d and their neighbours, the top of the range)."""
import numpy as np


def _magic(d):
    p = 0
    while (1 << p) < d:
        p += 1
    shift = 31 + p
    return (1 << shift) // d + 1, shift


def _check(d, ns):
    magic, shift = _magic(d)
    assert magic < (1 << 32)
    for n in ns:
        assert (n * magic) >> shift == n // d, (n, d)


def test_small_divisors_at_the_critical_numerators():
    top = (1 << 31) - 1
    for d in range(1, 4097):
        q = top // d
        ns = {0, 1, d - 1, d, d + 1, top, top - 1, q * d, q * d - 1, min(top, q * d + d - 1), (q // 2) * d - 1,
              (q // 2) * d}
        _check(d, [n for n in ns if 0 <= n <= top])


def test_large_and_random_divisors():
    rng = np.random.default_rng(0)
    top = (1 << 31) - 1
    ds = [int(v) for v in rng.integers(1, 1 << 31, size=400)] + [top, top - 1, 1 << 30, (1 << 30) + 1, (1 << 30) - 1,
                                                                  3136, 802816, 51380224, 11008, 65536, 16777216]
    for d in ds:
        q = top // d
        ns = [0, d - 1, d, top, q * d, max(0, q * d - 1)] + [int(v) for v in rng.integers(0, 1 << 31, size=50)]
        _check(d, [n for n in ns if 0 <= n <= top])
