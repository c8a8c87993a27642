"""The multiply-shift division the kernels use for row / channel indices, checked on the CPU:
q = umulhi(n, mul) >> shift with mul = ceil(2^(31+L) / d), shift = L - 1, L = ceil(log2 d)
must equal n // d for every n < 2^31 (the constants are restated from csrc/msd_device.h)."""
import numpy as np


def _consts(d):
    if d <= 1:
        return 0, 0
    L = 0
    while (1 << L) < d:
        L += 1
    return ((1 << (31 + L)) + d - 1) // d, L - 1


def test_fast_div_matches_integer_division():
    rng = np.random.default_rng(0)
    ns = np.concatenate([np.arange(0, 70000, dtype=np.uint64), rng.integers(0, 2 ** 31, 200000, dtype=np.uint64),
                         np.array([2 ** 31 - 1, 2 ** 31 - 2, 2 ** 30, 2 ** 30 - 1], dtype=np.uint64)])
    divisors = list(range(1, 700)) + [1023, 1024, 1025, 4095, 4096, 5120, 65535, 65536, 99991, 2 ** 20, 2 ** 24 + 1,
                                      2 ** 30, 2 ** 31 - 1]
    for d in divisors:
        mul, shift = _consts(d)
        assert mul < 2 ** 32
        q = ns if mul == 0 else ((ns * np.uint64(mul)) >> np.uint64(32)) >> np.uint64(shift)
        assert np.array_equal(q, ns // np.uint64(d)), d
