"""Pins the oracle's partition-id functions: against the reference's own packing, comparison and bit layout where the
reference library was built (oracle/_ref), against numpy's lower bound, and through the map's read-back."""
import numpy as np
import pytest

import oracle_lib
import texts


def test_bits_per_entry_match_the_reference_and_the_closed_form():
    ref = oracle_lib.ref()
    for p in list(range(1, 70)) + [255, 256, 257, 1023, 1024, 1025, 32768, 32769, 65535]:
        want = max(1, int(np.ceil(np.log2(p))) if p > 1 else 0) + 1
        assert oracle_lib.partition_id_bits(p) == want, p
        if ref is not None:
            assert ref.ref_partition_id_bits(p) == want, p


@pytest.mark.parametrize("bits", [2, 3, 5, 8, 9, 13, 16, 17])
def test_packing_matches_the_reference_group_by_group_and_reads_back(bits):
    rng = np.random.default_rng(bits)
    n = 64 * 5 + 37
    pid = rng.integers(0, 1 << (bits - 1), n).astype(np.uint16)
    pid[:4] = [(1 << (bits - 1)) - 1, 0, (1 << (bits - 1)) - 1, 1]
    got = oracle_lib.pack_partition_ids(pid, bits, fill=0xDEADBEEFDEADBEEF)
    assert got[oracle_lib.packed_words(n, bits):].tolist() == [0xDEADBEEFDEADBEEF] * (got.size - oracle_lib.packed_words(n, bits))
    for i in range(n):
        assert oracle_lib.oracle().orc_partition_id_map_get(got.ctypes.data, bits, i) == pid[i]
    # the layout by hand: entry i occupies bits [i * bits, (i + 1) * bits) of its group's words, flag bit clear
    for i in (0, 1, 63, 64, 100, n - 1):
        g, e = divmod(i, 64)
        val = 0
        for b in range(bits):
            bit = e * bits + b
            val |= ((int(got[g * bits + bit // 64]) >> (bit % 64)) & 1) << b
        assert val == pid[i]
    ref = oracle_lib.ref()
    if ref is not None:
        for off in range(0, n, 64):
            sz = min(64, n - off)
            dst = np.full(bits + 1, 0xDEADBEEFDEADBEEF, dtype=np.uint64)
            ref.ref_partition_id_pack(pid[off:].ctypes.data, sz, bits, dst.ctypes.data)
            nw = (sz * bits + 63) // 64
            assert np.array_equal(dst[:nw], got[(off // 64) * bits:(off // 64) * bits + nw]), off
            assert dst[nw] == 0xDEADBEEFDEADBEEF


@pytest.mark.parametrize("words", [1, 2, 3, 4])
@pytest.mark.parametrize("p", [1, 2, 3, 17, 300])
def test_ids_are_the_lower_bound_over_the_pivots(words, p):
    rng = np.random.default_rng(100 * words + p)
    T = texts.random_text(3000, 3, 9, sep_every=0)
    T[-9:] = 0
    pivots = oracle_lib.sample_pivots(T, p, words, rng, duplicates=True)
    pid, psz = oracle_lib.partition_ids(T, pivots, p, words)
    keys = oracle_lib.pack_prefix_np(T, words)
    # lexicographic lower bound by brute force on tuples
    kt = [tuple(int(v) for v in row) for row in keys]
    pt = [tuple(int(v) for v in row) for row in pivots]
    import bisect
    want = np.array([min(bisect.bisect_left(pt, k), p - 1) for k in kt], dtype=np.uint16)
    assert np.array_equal(pid, want)
    assert np.array_equal(psz, np.bincount(want, minlength=p).astype(np.uint64))
    if words == 1 and p > 1:
        assert np.array_equal(pid, np.minimum(np.searchsorted(pivots[:, 0], keys[:, 0], side="left"), p - 1))


def test_ids_satisfy_the_definition_under_the_references_own_comparison():
    ref = oracle_lib.ref()
    if ref is None:
        pytest.skip("the reference library was not built here")
    words = ref.ref_pivot_words()
    rng = np.random.default_rng(5)
    T = texts.random_text(2000, 2, 3, sep_every=0)
    padded = np.concatenate([T, np.zeros(4 * words, dtype=np.uint16)])  # the reference packs from a padded text
    for p in (2, 3, 40):
        pivots = oracle_lib.sample_pivots(T, p, words, rng, duplicates=True)
        pid, _ = oracle_lib.partition_ids(T, pivots, p, words)
        for i in range(T.size):
            q = int(pid[i])
            le = lambda k: bool(ref.ref_pivot_key_le_u16(padded[i:].ctypes.data, pivots[k].ctypes.data))
            assert q == p - 1 or le(q), (p, i)           # key <= pivots[q] unless q is the last partition
            assert q == 0 or not le(q - 1), (p, i)       # and q is the smallest such


def test_a_chunk_in_the_middle_of_the_text_sees_the_symbols_after_it():
    rng = np.random.default_rng(9)
    T = texts.random_text(1000, 4, 2, sep_every=0)
    words, p = 2, 9
    pivots = oracle_lib.sample_pivots(T, p, words, rng)
    whole, _ = oracle_lib.partition_ids(T, pivots, p, words)
    off, n = 128, 512
    chunk, _ = oracle_lib.partition_ids(T[off:], pivots, p, words, text_len=n + 4 * words - 1, n=n)
    assert np.array_equal(chunk, whole[off:off + n])


@pytest.mark.parametrize("generation0,ctx,key_words", [(True, 4, 1), (True, 8, 2), (False, 8, 1), (False, 64, 2)])
def test_staging_matches_the_references_tag_helpers(generation0, ctx, key_words):
    rng = np.random.default_rng(ctx + key_words)
    n, p = 700, 37
    T = texts.random_text(n, 5, 3, sep_every=0)
    pid = rng.integers(0, p, n).astype(np.uint16)
    retired = (rng.random(n) < 0.3).astype(np.uint8)
    suf = rng.permutation(n)[:300].astype(np.uint64)
    suf[:4] = [0, n - 1, ctx, max(ctx // 2 - 1, 0)]
    keys, beta = oracle_lib.stage_slab(T, suf, key_words, pid, retired, ctx, generation0)
    ell = 4 * key_words
    for i, j in enumerate(suf.tolist()):
        cur = 0 if j < ctx else int(pid[j - ctx]) | (0x8000 if retired[j - ctx] else 0)
        if generation0:
            prev = (int(pid[j + ell]) + ell) if j + ell < n else n + ell - 1 - (j + ell)
        else:
            prev = 0 if j < ctx // 2 else int(pid[j - ctx // 2]) | (0x8000 if retired[j - ctx // 2] else 0)
        assert beta[i] == ((prev & 0xFFFF) << 16 | cur), (i, j)
    if generation0:
        assert np.array_equal(keys, oracle_lib.pack_prefix_np(T, key_words)[suf.astype(np.int64)])
    ref = oracle_lib.ref()
    if ref is not None:
        for i, j in enumerate(suf.tolist()):
            assert beta[i] == ref.ref_beta_u16(j, n, ell, ctx, 1 if generation0 else 0, pid.ctypes.data, retired.ctypes.data), (i, j)
