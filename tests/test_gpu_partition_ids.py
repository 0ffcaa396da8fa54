"""Partition ids on the GPU (csa_partition_ids_u16_dev) against the oracle: ids, packed map and partition sizes."""
import numpy as np
import pytest

import oracle_lib
import texts

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    return torch


def dev16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint16).view(np.int16)).cuda()


def dev64(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint64).view(np.int64)).cuda()


def check(torch, T, pivots, p, words, tag):
    from cascade_amd import partition_ids
    print(f"  partition ids {tag} n={T.size} p={p} words={words}", flush=True)
    ids, packed, sizes = partition_ids(dev16(torch, T), dev64(torch, pivots).reshape(-1, words), p)
    torch.cuda.synchronize()
    want_ids, want_sizes = oracle_lib.partition_ids(T, pivots, p, words)
    bits = oracle_lib.partition_id_bits(p)
    assert np.array_equal(ids.cpu().numpy().view(np.uint16), want_ids), tag
    assert np.array_equal(sizes.cpu().numpy().view(np.uint64), want_sizes), tag
    want_packed = oracle_lib.pack_partition_ids(want_ids, bits)
    nw = oracle_lib.packed_words(T.size, bits)
    got = packed.cpu().numpy().view(np.uint64)
    assert np.array_equal(got[:nw], want_packed[:nw]), tag
    assert not got[nw:].any(), tag  # nothing is written past a trailing partial group


@pytest.mark.parametrize("words", [1, 2, 3, 4])
def test_ids_map_and_sizes_match_the_oracle(torch_mod, words):
    rng = np.random.default_rng(words)
    for n in (1, 63, 64, 65, 2047, 2048, 2049, 100003):
        T = texts.random_text(n, 3, n, sep_every=0)
        T[-min(n, 7):] = 0
        for p in (1, 2, 3, 17, 1000):
            check(torch_mod, T, oracle_lib.sample_pivots(T, p, words, rng, duplicates=True), p, words, f"n={n}")


@pytest.mark.parametrize("words", [2, 4])
def test_texts_whose_suffixes_start_like_the_pivots(torch_mod, words):
    """One symbol repeated, and separators only (K-grams of all ones, the value that pads the searched table): nearly every
    suffix equals some pivot in its first key word and is placed by the search over all words; pivot counts that fill the
    table exactly (p = 2^k) and that leave it padded."""
    rng = np.random.default_rng(10 + words)
    n = 70001
    for fill in (7, 0xFFFF):
        T = np.full(n, fill, dtype=np.uint16)
        T[n // 3] = 5
        T[n // 2:n // 2 + 40] = rng.integers(0, 3, 40)
        for p in (2, 16, 17, 256):
            check(torch_mod, T, oracle_lib.sample_pivots(T, p, words, rng, duplicates=True), p, words, f"fill={fill} p={p}")


def test_many_partitions_take_the_global_tables(torch_mod):
    # more pivots than fit in LDS, and more partitions than the LDS histogram holds
    rng = np.random.default_rng(3)
    T = rng.integers(0, 60000, 1 << 20).astype(np.uint16)
    for p, words in ((4097, 1), (4097, 2), (5000, 2), (65535, 2)):
        check(torch_mod, T, oracle_lib.sample_pivots(T, p, words, rng), p, words, "large p")


def test_zipf_tokens_at_sixteen_million(torch_mod):
    from cascade_amd import workloads
    rng = np.random.default_rng(4)
    T = workloads.generate(2, 1 << 24)
    check(torch_mod, T, oracle_lib.sample_pivots(T, 64, 2, rng), 64, 2, "C2 16M")


def test_chunks_add_up_to_the_whole_text(torch_mod):
    # the text in chunks that see 4 * words - 1 symbols past their end, sizes accumulated: same map, same sizes
    from cascade_amd import partition_ids
    torch = torch_mod
    rng = np.random.default_rng(6)
    words, p = 2, 33
    T = texts.random_text(50000, 4, 1, sep_every=0)
    pivots = oracle_lib.sample_pivots(T, p, words, rng)
    d_T, d_piv = dev16(torch, T), dev64(torch, pivots).reshape(-1, words)
    want_ids, want_sizes = oracle_lib.partition_ids(T, pivots, p, words)
    sizes = torch.zeros(p, dtype=torch.int64, device="cuda")
    got = []
    chunk = 64 * 200
    for off in range(0, T.size, chunk):
        n = min(chunk, T.size - off)
        tl = min(n + 4 * words - 1, T.size - off)
        ids, _, _ = partition_ids(d_T[off:], d_piv, p, n=n, text_len=tl, want_packed=False, sizes=sizes)
        got.append(ids.cpu().numpy().view(np.uint16))
    assert np.array_equal(np.concatenate(got), want_ids)
    assert np.array_equal(sizes.cpu().numpy().view(np.uint64), want_sizes)


def test_text_pointer_at_every_alignment(torch_mod):
    from cascade_amd import partition_ids
    torch = torch_mod
    rng = np.random.default_rng(8)
    backing = torch.zeros(9000, dtype=torch.int16, device="cuda")
    for off in range(4):
        n = 5000 + off
        T = rng.integers(0, 3, n).astype(np.uint16)
        window = backing[off:off + n]
        window.copy_(torch.from_numpy(T.view(np.int16)))
        pivots = oracle_lib.sample_pivots(T, 9, 2, rng)
        ids, _, _ = partition_ids(window, dev64(torch, pivots).reshape(-1, 2), 9, want_packed=False, want_sizes=False)
        assert np.array_equal(ids.cpu().numpy().view(np.uint16), oracle_lib.partition_ids(T, pivots, 9, 2)[0]), off


def test_bad_arguments_are_refused(torch_mod):
    from cascade_amd import _native
    lib = _native.load()
    assert lib.csa_partition_ids_u16_dev(None, 10, 10, None, 2, 0, None, None, None, None) == _native.CSA_ERR_ARG
    assert lib.csa_partition_ids_u16_dev(None, 10, 10, None, 5, 3, None, None, None, None) == _native.CSA_ERR_ARG
    assert lib.csa_partition_ids_u16_dev(None, 10, 5, None, 2, 1, None, None, None, None) == _native.CSA_ERR_ARG
    assert lib.csa_partition_ids_u16_dev(None, 0, 0, None, 2, 3, None, None, None, None) == _native.CSA_OK


@pytest.mark.parametrize("generation0,ctx,key_words", [(True, 4, 1), (True, 8, 2), (False, 8, 1), (False, 4096, 2)])
def test_slab_staging_on_the_device_matches_the_oracle(torch_mod, generation0, ctx, key_words):
    # the packed map comes from the partition-id kernel itself; some suffixes are then marked retired
    from cascade_amd import partition_ids, stage_slab
    torch = torch_mod
    rng = np.random.default_rng(ctx)
    n, p = 300000, 29
    T = texts.random_text(n, 6, 1, sep_every=0)
    pivots = oracle_lib.sample_pivots(T, p, 2, rng)
    d_T = dev16(torch, T)
    ids, packed, _ = partition_ids(d_T, dev64(torch, pivots).reshape(-1, 2), p)
    pid = ids.cpu().numpy().view(np.uint16)
    bits = oracle_lib.partition_id_bits(p)
    words = packed.cpu().numpy().view(np.uint64).copy()
    retired = (rng.random(n) < 0.25).astype(np.uint8)
    oracle_lib.set_retired(words, bits, np.flatnonzero(retired))
    suf = rng.permutation(n)[:100000].astype(np.uint64)
    suf[:6] = [0, 1, n - 1, n - 2, ctx, max(ctx // 2 - 1, 0)]
    lanes = oracle_lib.u64_to_sa40(suf)
    print(f"  stage n={n} count={suf.size} ctx={ctx} gen0={generation0}", flush=True)
    keys, beta = stage_slab(d_T, torch.from_numpy(lanes).cuda(), key_words, dev64(torch, words), p, ctx, generation0)
    want_keys, want_beta = oracle_lib.stage_slab(T, suf, key_words, pid, retired, ctx, generation0)
    assert np.array_equal(beta.cpu().numpy().view(np.uint32), want_beta)
    if generation0:
        assert np.array_equal(keys.cpu().numpy().view(np.uint64), want_keys)
