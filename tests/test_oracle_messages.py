"""Pins the oracle's message functions against the reference's own bit helpers (oracle/_ref) and against their
definitions worked out with numpy."""
import numpy as np
import pytest

import message_cases
import oracle_lib


@pytest.mark.parametrize("packed,ctx", [(False, 4), (True, 8), (True, 4096)])
def test_messages_of_agrees_with_the_reference_helpers(packed, ctx):
    ref = oracle_lib.ref()
    if ref is None:
        pytest.skip("the reference library was not built here")
    sa, keys, beta, active_sz = message_cases.cohort(3000, 50, ctx, packed, seed=ctx)
    a, b = np.zeros(6, dtype=np.uint64), np.zeros(6, dtype=np.uint64)
    kinds = set()
    for i in range(sa.size):
        oracle_lib.oracle().orc_messages_of(int(sa[i]), int(keys[i]), int(beta[i]), i, active_sz, ctx, int(packed), a.ctypes.data)
        ref.ref_messages_of(int(sa[i]), int(keys[i]), int(beta[i]), i, active_sz, ctx, int(packed), b.ctypes.data)
        assert np.array_equal(a, b), i
        kinds.add((a[0] != 0xFFFFFFFF, a[3] != 0xFFFFFFFF))
    assert len(kinds) == (4 if packed else 2)  # every combination of payload / forwarded pill occurred


def test_counts_and_emission_follow_the_definition():
    p, ctx = 13, 16
    sa, keys, beta, active_sz = message_cases.cohort(5000, p, ctx, True, seed=1)
    j = sa & np.uint64((1 << 48) - 1)
    pay = (j >= ctx) & ((beta & 0x8000) == 0)
    fwd = ((keys >> np.uint64(62)) & np.uint64(1)).astype(bool) & (j >= ctx // 2) & (((beta >> 16) & 0x8000) == 0)
    want = np.bincount(beta[pay] & 0xFFFF, minlength=p + 1) + np.bincount(beta[fwd] >> 16, minlength=p + 1)
    cnt = oracle_lib.count_messages(sa, keys, beta, ctx, True, p)
    assert np.array_equal(cnt, want.astype(np.uint32))
    tgt, rank, end = oracle_lib.emit_messages(sa, keys, beta, ctx, True, active_sz, p)
    assert np.array_equal(end[:p], np.cumsum(cnt[:p]))  # every counter ends at its group's end
    got = message_cases.groups(tgt, rank, end, p)
    idx = np.arange(sa.size)
    for q in range(p):
        m = pay & ((beta & 0xFFFF) == q)
        r = ((keys[m] >> np.uint64(31)) & np.uint64(0x7FFFFFFF)).astype(np.uint32) | (np.uint32(1 << 31) * (idx[m] >= active_sz))
        exp = list(zip((j[m] - np.uint64(ctx)).tolist(), r.tolist()))
        m2 = fwd & ((beta >> 16) == q)
        r2 = (keys[m2] & np.uint64(0x7FFFFFFF)).astype(np.uint32) | np.uint32(1 << 31)
        exp += list(zip((j[m2] - np.uint64(ctx // 2)).tolist(), r2.tolist()))
        assert got[q] == sorted(exp), q


def test_join_delivers_to_cohort_members_and_drops_the_rest():
    rng = np.random.default_rng(2)
    n = 4000
    suf = np.sort(rng.choice(1 << 20, n, replace=False)).astype(np.uint64)
    sa = suf | (rng.integers(0, 1 << 16, n).astype(np.uint64) << np.uint64(48))
    primary = rng.integers(0, 1 << 31, n).astype(np.uint32)
    hit = rng.choice(n, 1500, replace=False)
    miss = np.setdiff1d(rng.integers(0, 1 << 20, 500).astype(np.uint64), suf)
    tgt = np.concatenate([suf[hit], miss])
    rank = rng.integers(0, 1 << 32, tgt.size, dtype=np.uint64).astype(np.uint32)
    order = rng.permutation(tgt.size)
    tgt, rank = tgt[order], rank[order]
    seed_keys = np.full(n, np.uint64(0xFFFFFFFFFFFFFFFF))  # "no message joined" (src/GPU_SACA.cu:1825-1826)
    keys = oracle_lib.join_messages(tgt, rank, sa, primary, seed_keys)
    want = seed_keys.copy()
    pos = np.searchsorted(suf, tgt)
    ok = (pos < n) & (suf[np.minimum(pos, n - 1)] == tgt)
    r = rank[ok].astype(np.uint64)
    want[pos[ok]] = (primary[pos[ok]].astype(np.uint64) << np.uint64(31)) | (r & np.uint64(0x7FFFFFFF)) | ((r >> np.uint64(31)) << np.uint64(62))
    assert np.array_equal(keys, want) and ok.sum() == 1500
    ref = oracle_lib.ref()
    if ref is not None:
        for q, rr in zip(pos[ok][:300].tolist(), rank[ok][:300].tolist()):
            assert int(keys[q]) == ref.ref_joined_key(int(primary[q]), rr)
