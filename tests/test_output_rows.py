"""The step after the partition sort: the cuts of a partition's output range (host arithmetic, runs anywhere) and, on the
GPU, the rank-order scatter of (suffix, rank) pairs into 5-byte lanes."""
import numpy as np
import pytest

import oracle_lib

BLK = 4096


def cuts_of(fn, lo, hi, chunk_bytes, chunk_c):
    return [fn(lo, hi, chunk_bytes, c, chunk_c) for c in range(chunk_c)]


def check_cut_properties(cuts, lo, hi, chunk_bytes):
    """What the cuts are for (src/Output_File.cpp:18-35, include/Output_File.hpp:23-37): together they tile [lo, hi) exactly;
    every piece is whole disk blocks inside its chunk's window; only the first chunk has a head and only the last a tail."""
    covered = []
    base = lo // BLK * BLK
    for c, (plo, phi, hlo, hhi, tlo, thi) in enumerate(cuts):
        assert plo <= phi and plo % BLK == 0 and phi % BLK == 0
        if plo < phi:
            assert base + c * chunk_bytes <= plo and phi <= base + (c + 1) * chunk_bytes
            covered.append((plo, phi))
        if c != 0:
            assert hlo == hhi
        if c != len(cuts) - 1:
            assert tlo == thi
        if hlo < hhi:
            covered.append((hlo, hhi))
        if tlo < thi:
            covered.append((tlo, thi))
    covered.sort()
    pos = lo
    for a, b in covered:
        assert a == pos, (covered, lo, hi)
        pos = b
    assert pos == hi or (lo == hi and not covered)


def test_cut_known_answers_and_properties():
    from cascade_amd import output_cut
    # a range of 5-byte lanes that starts and ends inside blocks, three chunks of two blocks
    lo, hi, cb = 5 * 1000, 5 * 1000 + 5 * 5000, 2 * BLK
    want = [(8192, 12288, 5000, 8192, 0, 0), (12288, 20480, 0, 0, 0, 0), (20480, 28672, 0, 0, 28672, 30000)]
    assert cuts_of(output_cut, lo, hi, cb, 3) == want
    assert [tuple(oracle_lib.output_cut(lo, hi, cb, c, 3)) for c in range(3)] == want
    # a range inside one block: all head
    assert output_cut(100, 200, BLK, 0, 1) == (4096, 4096, 100, 200, 4096, 4096)
    rng = np.random.default_rng(0)
    for _ in range(2000):
        lo = int(rng.integers(0, 1 << 20))
        hi = lo + int(rng.integers(0, 1 << 18))
        cb = BLK * int(rng.integers(1, 9))
        chunk_c = max(1, -(-(hi - lo // BLK * BLK) // cb))
        got = cuts_of(output_cut, lo, hi, cb, chunk_c)
        assert got == [tuple(oracle_lib.output_cut(lo, hi, cb, c, chunk_c)) for c in range(chunk_c)]
        check_cut_properties(got, lo, hi, cb)


def test_oracle_scatter_is_the_inverse_permutation():
    rng = np.random.default_rng(1)
    m = 1000
    suf = rng.integers(0, 1 << 40, m).astype(np.uint64)
    rank = rng.permutation(m).astype(np.uint32)
    rc, out = oracle_lib.scatter_to_rank_order(oracle_lib.u64_to_sa40(suf)[:5 * m], rank)
    want = np.zeros(m, dtype=np.uint64)
    want[rank] = suf
    assert rc == 0 and np.array_equal(oracle_lib.sa40_to_u64(out), want)
    rank[3] = m
    assert oracle_lib.scatter_to_rank_order(oracle_lib.u64_to_sa40(suf)[:5 * m], rank)[0] == -1


@pytest.mark.gpu
@pytest.mark.parametrize("m,capacity", [(1, 16), (5, 16), (255, 16), (256, 16), (257, 16), (100003, 16), (1 << 22, 16),
                                        ((1 << 25) + 12345, (1 << 25) + 12345), (1 << 26, 1 << 27)])
def test_gpu_scatter_to_rank_order_matches_the_oracle(m, capacity):
    """A handle smaller than the partition scatters directly; one that holds it buckets large partitions by windows of
    the output first (same result)."""
    import torch
    from cascade_amd import PartitionSorter, _native
    rng = np.random.default_rng(m)
    suf = rng.integers(0, 1 << 40, m).astype(np.uint64)
    rank = rng.permutation(m).astype(np.uint32)
    lanes = oracle_lib.u64_to_sa40(suf)[:5 * m]
    s = PartitionSorter(capacity)
    try:
        print(f"  scatter m={m} capacity={capacity}", flush=True)
        out = s.scatter_to_rank_order(torch.from_numpy(lanes).cuda(), torch.from_numpy(rank.view(np.int32)).cuda())
        assert np.array_equal(out.cpu().numpy(), oracle_lib.scatter_to_rank_order(lanes, rank)[1])
        if m > 5:
            rank[m // 2] = m  # out of range: refused, nothing written out of bounds
            with pytest.raises(_native.CascadeError):
                s.scatter_to_rank_order(torch.from_numpy(lanes).cuda(), torch.from_numpy(rank.view(np.int32)).cuda())
    finally:
        s.close()
