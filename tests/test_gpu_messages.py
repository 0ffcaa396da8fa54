"""Message kernels on the GPU (count, offsets, emit, join) against the oracle, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

import message_cases
import oracle_lib

pytestmark = pytest.mark.gpu


def run_messages(lib, to_dev, to_host, sa, keys, beta, ctx, packed, active_sz, p):
    """count -> offsets -> emit through `lib`; returns (counts, targets, ranks, end offsets)."""
    n = sa.size
    d_sa, d_keys, d_beta = to_dev(sa), to_dev(keys), to_dev(beta)
    d_cnt = to_dev(np.zeros(p + 1, dtype=np.uint32))
    assert lib.csa_count_messages_dev(d_sa.ptr, d_keys.ptr, d_beta.ptr, n, ctx, int(packed), p, d_cnt.ptr, None) == 0
    cnt = to_host(d_cnt)
    assert lib.csa_message_offsets_dev(d_cnt.ptr, p + 1, None) == 0
    start = to_host(d_cnt)
    total = int(cnt.sum())
    d_tgt = to_dev(np.zeros(5 * max(total, 1), dtype=np.uint8))
    d_rank = to_dev(np.zeros(max(total, 1), dtype=np.uint32))
    d_act = to_dev(np.array([active_sz], dtype=np.uint64))
    assert lib.csa_emit_messages_dev(d_sa.ptr, d_keys.ptr, d_beta.ptr, n, ctx, int(packed), d_act.ptr, p, d_tgt.ptr, d_rank.ptr,
                                     d_cnt.ptr, None) == 0
    return cnt, start, oracle_lib.sa40_to_u64(to_host(d_tgt))[:total], to_host(d_rank)[:total], to_host(d_cnt)


def check_messages(lib, to_dev, to_host, n, p, ctx, packed, seed):
    sa, keys, beta, active_sz = message_cases.cohort(n, p, ctx, packed, seed)
    cnt, start, tgt, rank, end = run_messages(lib, to_dev, to_host, sa, keys, beta, ctx, packed, active_sz, p)
    want_cnt = oracle_lib.count_messages(sa, keys, beta, ctx, packed, p)
    assert np.array_equal(cnt, want_cnt)
    assert np.array_equal(start[1:], np.cumsum(want_cnt[:-1])) and start[0] == 0
    w_tgt, w_rank, w_end = oracle_lib.emit_messages(sa, keys, beta, ctx, packed, active_sz, p)
    assert np.array_equal(end, w_end)
    assert message_cases.groups(tgt, rank, end, p) == message_cases.groups(w_tgt, w_rank, w_end, p)


class DevArray:
    def __init__(self, tensor):
        self.t = tensor
        self.ptr = tensor.data_ptr()


@pytest.fixture(scope="module")
def gpu():
    import torch
    from cascade_amd import _native
    assert torch.cuda.is_available()
    view = {np.dtype(np.uint64): np.int64, np.dtype(np.uint32): np.int32, np.dtype(np.uint8): np.uint8}

    def to_dev(a):
        a = np.ascontiguousarray(a)
        return DevArray(torch.from_numpy(a.view(view[a.dtype])).cuda())

    def to_host(d):
        torch.cuda.synchronize()
        a = d.t.cpu().numpy()
        return a.view({np.dtype(np.int64): np.uint64, np.dtype(np.int32): np.uint32, np.dtype(np.uint8): np.uint8}[a.dtype])

    return _native.load(), to_dev, to_host


@pytest.mark.parametrize("packed,ctx", [(False, 4), (True, 8), (True, 1 << 20)])
def test_count_offsets_and_emit_match_the_oracle(gpu, packed, ctx):
    lib, to_dev, to_host = gpu
    for n, p in ((1, 3), (255, 3), (1025, 17), (100003, 64), (70001, 256), (70001, 257), (1 << 20, 2048), (50000, 2049), (50000, 32768)):
        print(f"  messages n={n} p={p} ctx={ctx} packed={packed}", flush=True)
        check_messages(lib, to_dev, to_host, n, p, ctx, packed, seed=n + p)


def test_join_matches_the_oracle(gpu):
    lib, to_dev, to_host = gpu
    rng = np.random.default_rng(3)
    for n, hits, misses in ((1, 1, 3), (1000, 400, 100), (1 << 20, 300000, 50000), (200001, 5000, 3000), (150000, 60, 40)):
        if n == 200001:    # 40-bit suffixes in two far-apart clusters: most buckets of the join's directory are empty
            suf = np.unique(np.concatenate([rng.integers(0, 1 << 20, n // 2), (1 << 40) - 1 - rng.integers(0, 1 << 22, n // 2)])
                            .astype(np.uint64))
            n = suf.size
        elif n == 150000:  # few messages: the handle of the sorted variant has room for a small directory only
            suf = np.sort(rng.choice(1 << 36, n, replace=False)).astype(np.uint64)
        else:
            suf = np.sort(rng.choice(1 << 30, n, replace=False)).astype(np.uint64)
        sa = suf | (rng.integers(0, 1 << 16, n).astype(np.uint64) << np.uint64(48))
        primary = rng.integers(0, 1 << 31, n).astype(np.uint32)
        tgt = np.concatenate([suf[rng.choice(n, hits, replace=False)],
                              np.setdiff1d(rng.integers(0, int(suf[-1]) + 1000, misses).astype(np.uint64), suf)])
        rank = rng.integers(0, 1 << 32, tgt.size, dtype=np.uint64).astype(np.uint32)
        order = rng.permutation(tgt.size)
        tgt, rank = tgt[order], rank[order]
        seed_keys = np.full(n, np.uint64(0xFFFFFFFFFFFFFFFF))
        d_keys = to_dev(seed_keys)
        print(f"  join n={n} messages={tgt.size}", flush=True)
        d_tgt, d_rank, d_sa, d_primary = to_dev(oracle_lib.u64_to_sa40(tgt)), to_dev(rank), to_dev(sa), to_dev(primary)  # kept alive
        assert lib.csa_join_messages_dev(d_tgt.ptr, d_rank.ptr, tgt.size, d_sa.ptr, d_primary.ptr, d_keys.ptr, n, None) == 0
        want = oracle_lib.join_messages(tgt, rank, sa, primary, seed_keys)
        assert np.array_equal(to_host(d_keys), want)
        # the same through the variant that sorts the inbox by target first (scratch of a handle)
        from cascade_amd import PartitionSorter
        with PartitionSorter(max(tgt.size, 16)) as s:
            d_keys2 = to_dev(seed_keys)
            d_lanes = to_dev(oracle_lib.u64_to_sa40(tgt))
            assert lib.csa_join_messages_sorted_dev(s._h, d_lanes.ptr, d_rank.ptr, tgt.size, d_sa.ptr, d_primary.ptr, d_keys2.ptr, n,
                                                    None) == 0
            assert np.array_equal(to_host(d_keys2), want)
            assert np.array_equal(to_host(d_lanes), oracle_lib.u64_to_sa40(tgt))  # the inbox is left alone
