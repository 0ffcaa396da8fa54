"""Seeded input texts shared by the oracle tests and the GPU parity tests (numpy PCG64, portable)."""
import numpy as np

SEP = 0xFFFF


def random_text(n, sigma, seed, sep_every=50):
    """n uint16 symbols over an alphabet of `sigma` values spread over [0, 65535] (0 and the maximum included),
    with separators 0xFFFF about every `sep_every` symbols: the shape of the reference's random fixtures
    (src/test_query.cu:317-331)."""
    rng = np.random.default_rng(seed)
    if sigma == 65536:
        alpha = np.arange(65536, dtype=np.uint64)
    else:
        alpha = (np.arange(sigma, dtype=np.uint64) * 65535) // max(sigma - 1, 1)
    T = alpha[rng.integers(0, len(alpha), size=n)].astype(np.uint16)
    if sep_every:
        T[rng.random(n) < 1.0 / sep_every] = SEP
    return T


def periodic(k=3000, a=3, b=7):
    return np.array([b if i % 2 else a for i in range(k)], dtype=np.uint16)


def fibonacci_word(min_len=2500):
    fib, prev = [1], [0]
    while len(fib) < min_len:
        fib, prev = fib + prev, fib
    return np.array(fib, dtype=np.uint16)


def hand_cases():
    """Texts of the reference's edge cases (src/test_query.cu:374-392) plus tail-rule corner cases."""
    cases = [
        [0, 0, 0, 0], [5, 3, 5, 0], [9, 8, 7], [3, 4, 5], [65535, 1, 65535, 1, 65535], [65535, 65535],
        [0], [7], [0, 0], [1, 0], [0, 1], [0, 0, 0], [0, 0, 0, 0, 0], [0] * 9, [0] * 17, [5, 0, 0, 0, 0, 5, 0, 0, 0],
        [5, 0, 0, 0, 5, 0, 0, 0], [1, 2, 3, 4, 1, 2, 3, 4, 1, 2, 3, 4], [1, 2, 3, 0, 0, 0, 0, 1, 2, 3, 0, 0, 0],
        [2, 1, 0, 0, 0, 0, 0, 0, 0, 0, 2, 1, 0, 0, 0, 0], list(range(20)), list(range(20, 0, -1)),
        [4] * 33, [0, 0, 0, 0, 0, 0, 0, 0, 1], [1, 0, 0, 0, 0, 0, 0, 0, 0],
    ]
    return [np.array(c, dtype=np.uint16) for c in cases]


def zero_tail_corner(n=5000, ell=4, seed=9):
    """Random text over a tiny alphabet ending in a run of zeros: the missing-terminator corner case
    (dataset/make-corner-case.py) whose expected first entries are n-1, n-2, ..., n-ell."""
    rng = np.random.default_rng(seed)
    T = rng.integers(0, 3, size=n).astype(np.uint16)
    T[-(ell + 3):] = 0
    return T


def fixture_suite():
    """(name, text) pairs used for golden vectors and parity."""
    out = []
    i = 0
    for n in (1, 2, 3, 15, 16, 17, 1000, 8000):
        for sigma in (2, 3, 4, 16, 256, 65536):
            out.append((f"rand_n{n}_s{sigma}", random_text(n, sigma, 1000 + i)))
            i += 1
    out.append(("periodic_ab", periodic()))
    out.append(("fibonacci", fibonacci_word()))
    out.append(("zero_tail", zero_tail_corner()))
    for k, c in enumerate(hand_cases()):
        out.append((f"hand_{k}", c))
    return out
