"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real MI355X."""
import hashlib
import os

import numpy as np
import pytest

import oracle_lib
import texts

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    return torch


# Every test that sorts through these handles runs twice: with the default tile order of the radix passes (tiles numbered
# by arrival) and with the XCD-chunked order a caller gets after csa_set_device_exclusive (the order the headline
# benchmark figure is measured with). Both must give the oracle's bytes.
TILE_ORDERS = pytest.mark.parametrize("exclusive", [False, True], ids=["tiles_by_arrival", "tiles_xcd_chunked"])


@pytest.fixture(scope="module", params=[False, True], ids=["tiles_by_arrival", "tiles_xcd_chunked"])
def sorter(torch_mod, request):
    from cascade_amd import PartitionSorter
    s = PartitionSorter(1 << 22, key_words=1, device_exclusive=request.param)
    yield s
    s.close()


@pytest.fixture(scope="module", params=[False, True], ids=["tiles_by_arrival", "tiles_xcd_chunked"])
def sorter2(torch_mod, request):
    from cascade_amd import PartitionSorter
    s = PartitionSorter(1 << 21, key_words=2, device_exclusive=request.param)
    yield s
    s.close()


def to_dev(torch, a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda()
    if a.dtype == np.uint64:
        return torch.from_numpy(a.view(np.int64)).cuda()
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    return torch.from_numpy(a).cuda()


def gpu_sa40(torch, s, T, index_base=0):
    print(f"  sort n={len(T)} key_words={s.key_words}", flush=True)
    d = to_dev(torch, np.asarray(T, dtype=np.uint16))
    out = s.sort(d, index_base=index_base)
    torch.cuda.synchronize()
    return out.cpu().numpy()


# ---- stage: K-gram key packing ---------------------------------------------------------------------

@pytest.mark.parametrize("key_words", [1, 2, 3, 4])
def test_pack_keys_matches_oracle(torch_mod, key_words):
    from cascade_amd import pack_keys
    for n, sigma, seed in ((1, 4, 0), (3, 4, 1), (4, 4, 2), (5, 65536, 3), (1000, 65536, 4), (100003, 65536, 5)):
        T = texts.random_text(n, sigma, seed)
        got = pack_keys(to_dev(torch_mod, T), key_words).cpu().numpy().view(np.uint64)
        want = oracle_lib.pack_prefix_np(T, key_words)
        assert np.array_equal(got, want), (n, key_words)


# ---- stage: radix sort -----------------------------------------------------------------------------

@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 8191, 8192, 8193, 100000, 1 << 20])
def test_radix_sort_pairs_matches_stable_sort(torch_mod, sorter, n):
    rng = np.random.default_rng(n)
    keys = rng.integers(0, 1 << 63, n, dtype=np.uint64) * np.uint64(2) + rng.integers(0, 2, n, dtype=np.uint64)
    vals = np.arange(n, dtype=np.uint32)
    dk, dv = to_dev(torch_mod, keys), to_dev(torch_mod, vals)
    sorter.radix_sort_pairs(dk, dv)
    wk, wv = oracle_lib.stable_sort_pairs(keys, vals)
    assert np.array_equal(dk.cpu().numpy().view(np.uint64), wk)
    assert np.array_equal(dv.cpu().numpy().view(np.uint32), wv)


def test_radix_sort_is_stable_on_skewed_keys_and_bit_ranges(torch_mod, sorter):
    rng = np.random.default_rng(3)
    n = 300000
    cases = [
        (rng.integers(0, 4, n).astype(np.uint64), 0, 64),                       # four values: long runs of ties
        (np.zeros(n, dtype=np.uint64), 0, 64),                                  # every pass trivial
        (np.full(n, 0xFFFFFFFFFFFFFFFF, dtype=np.uint64), 0, 64),               # collides with the tile padding
        (rng.zipf(1.3, n).astype(np.uint64) << np.uint64(13), 13, 40),          # a bit sub-range
        (rng.integers(0, 1 << 30, n).astype(np.uint64) | (rng.integers(0, 7, n).astype(np.uint64) << np.uint64(30)), 0, 33),
        (np.where(rng.random(n) < 0.5, np.uint64(0xFF), np.uint64(0xFFFF)).astype(np.uint64), 0, 16),
    ]
    for keys, b, e in cases:
        vals = rng.permutation(n).astype(np.uint32)
        dk, dv = to_dev(torch_mod, keys), to_dev(torch_mod, vals)
        sorter.radix_sort_pairs(dk, dv, b, e)
        wk, wv = oracle_lib.stable_sort_pairs(keys, vals, b, e)
        assert np.array_equal(dk.cpu().numpy().view(np.uint64), wk)
        assert np.array_equal(dv.cpu().numpy().view(np.uint32), wv)


# ---- whole partition: golden vectors of the reference's CPU sort ----------------------------------------

def test_golden_fixtures_bit_exact(torch_mod, sorter, sorter2):
    g = np.load(os.path.join(GOLDEN, "fixtures.npz"), allow_pickle=False)
    for name, T in texts.fixture_suite():
        want = g[f"{name}.sa40"]
        for s in (sorter, sorter2):
            got = gpu_sa40(torch_mod, s, T)
            assert got.dtype == np.uint8 and got.size == 5 * len(T)
            assert np.array_equal(got, want), f"{name} key_words={s.key_words}"


def test_empty_partition(torch_mod, sorter):
    d = torch_mod.empty(0, dtype=torch_mod.int16, device="cuda")
    out = sorter.sort(d)
    assert out.numel() == 0 and sorter.last_stats["generations"] == 0


def test_c1_matches_reference_digest_and_generation_counts(torch_mod, sorter):
    from cascade_amd import workloads
    want = dict(line.split() for line in open(os.path.join(GOLDEN, "c1_sha256.txt")))
    T = workloads.generate(1)
    got = gpu_sa40(torch_mod, sorter, T)
    assert hashlib.sha256(got.tobytes()).hexdigest() == want["sa40"]
    _, counts = oracle_lib.prefix_doubling(T, 1)
    assert sorter.last_stats["active"] == counts  # suffixes active entering each generation


@pytest.mark.parametrize("config,n", [(2, 1 << 20), (3, 1 << 21), (4, 1 << 20), (5, 1 << 20)])
def test_scaled_configs_against_oracle(torch_mod, sorter, config, n):
    from cascade_amd import workloads
    T = workloads.generate(config, n)
    got = gpu_sa40(torch_mod, sorter, T)
    sa, counts = oracle_lib.prefix_doubling(T, 1)
    assert np.array_equal(got, oracle_lib.u64_to_sa40(sa))
    assert sorter.last_stats["active"] == counts
    assert oracle_lib.is_correct_sa40(got, T)


def test_key_words_2_on_deep_repeats(torch_mod, sorter2):
    from cascade_amd import workloads
    for config in (3, 5):
        T = workloads.generate(config, 1 << 19)
        got = gpu_sa40(torch_mod, sorter2, T)
        sa, counts = oracle_lib.prefix_doubling(T, 2)
        assert np.array_equal(got, oracle_lib.u64_to_sa40(sa))
        assert sorter2.last_stats["active"] == counts


def test_index_base_offsets_every_entry(torch_mod, sorter):
    T = texts.random_text(5000, 4, 11)
    base = (1 << 39) + 12345
    a = oracle_lib.sa40_to_u64(gpu_sa40(torch_mod, sorter, T))
    b = oracle_lib.sa40_to_u64(gpu_sa40(torch_mod, sorter, T, index_base=base))
    assert np.array_equal(a + np.uint64(base), b)


def test_device_verifier_agrees_with_oracle(torch_mod, sorter):
    T = texts.random_text(20000, 3, 21)
    d = to_dev(torch_mod, T)
    out = sorter.sort(d).clone()
    assert sorter.verify(d, out)
    sa = oracle_lib.sa40_to_u64(out.cpu().numpy())
    for mutate in ("swap", "oob", "repeat"):
        bad = sa.copy()
        if mutate == "swap":
            bad[[100, 101]] = bad[[101, 100]]
        elif mutate == "oob":
            bad[7] = len(T) + 3
        else:
            bad[11] = bad[10]
        assert not oracle_lib.is_correct_sa(bad, T)
        assert not sorter.verify(d, to_dev(torch_mod, oracle_lib.u64_to_sa40(bad)))


def test_host_buffer_entry_point_and_file_interface(torch_mod, tmp_path):
    from cascade_amd import GPU_SACA, sort_partition
    T = texts.random_text(30000, 16, 5)
    sa40, stats = sort_partition(T, 1)
    assert np.array_equal(sa40, oracle_lib.build_sa40(T)) and stats["n"] == len(T)
    ip, op = tmp_path / "text.u16", tmp_path / "sa.bin"
    T.astype("<u2").tofile(ip)
    GPU_SACA(str(ip), str(op)).build_SA()
    assert np.array_equal(np.fromfile(op, dtype=np.uint8), sa40)


def test_pipelined_host_buffer_entry_sorts_every_partition_of_a_list(torch_mod):
    """csa_sort_partitions_u16: partitions of different sizes (an empty one among them) from pinned and from pageable host
    memory, with index bases, each byte-equal to the oracle's sort; the upload and download threads must hand every
    buffer over at the right time."""
    from cascade_amd import sort_partitions, workloads
    rng = np.random.default_rng(8)
    sizes = [70000, 1, 0, 300000, 5000, 123457, 2, 99999, 150000]
    texts_k = [workloads.generate(3 if k % 2 else 5, n) if n >= 64 else rng.integers(0, 3, n).astype(np.uint16) for k, n in enumerate(sizes)]
    bases = [int(rng.integers(0, 1 << 39)) for _ in sizes]
    for pinned in (False, True):
        ins, outs = texts_k, None
        if pinned:
            keep = [torch_mod.from_numpy(t.view(np.int16).copy()).pin_memory() for t in texts_k]
            ins = [k.numpy().view(np.uint16) for k in keep]
            outs = [torch_mod.empty(max(5 * t.size, 1), dtype=torch_mod.uint8, pin_memory=True).numpy() for t in texts_k]
        print(f"  pipelined host entry, {len(sizes)} partitions, pinned={pinned}", flush=True)
        got, stats = sort_partitions(ins, key_words=1, index_base=bases, out=outs)
        for k, T in enumerate(texts_k):
            want = oracle_lib.sa40_to_u64(oracle_lib.build_sa40(T)) + np.uint64(bases[k])
            assert np.array_equal(oracle_lib.sa40_to_u64(got[k]), want), (k, T.size, pinned)
            assert stats[k]["n"] == T.size


def test_text_pointer_at_every_alignment(torch_mod, sorter, sorter2):
    # the text may start anywhere inside an aligned 8-byte word (a window of a larger buffer), and end anywhere too
    torch = torch_mod
    rng = np.random.default_rng(11)
    backing = torch.zeros(40000, dtype=torch.int16, device="cuda")
    for off in range(4):
        for n in (20001 + off, 24576, 8193 - off):
            T = rng.integers(0, 3, n).astype(np.uint16)
            T[-6:] = 0
            window = backing[off:off + n]
            window.copy_(torch.from_numpy(T.view(np.int16)))
            assert window.data_ptr() % 8 == 2 * off
            want = oracle_lib.build_sa40(T)
            for s in (sorter, sorter2):
                print(f"  sort off={off} n={n} key_words={s.key_words}", flush=True)
                got = s.sort(window).cpu().numpy()
                assert np.array_equal(got, want), (off, n, s.key_words)


def test_repeatable(torch_mod, sorter):
    from cascade_amd import workloads
    T = workloads.generate(5, 1 << 18)
    a = gpu_sa40(torch_mod, sorter, T)
    b = gpu_sa40(torch_mod, sorter, T)
    assert np.array_equal(a, b)


def test_many_small_partitions_of_low_entropy(torch_mod):
    """Low-entropy texts around the tile sizes of the kernels (2048 and 8192): large groups, groups that straddle
    tiles, several generations. Fresh handles sized exactly to the partition, so any index out of range shows."""
    from cascade_amd import PartitionSorter
    rng = np.random.default_rng(2024)
    for n in (2047, 2048, 2049, 4100, 8000, 8191, 8192, 8193, 12000, 20000, 50000):
        for sigma in (2, 3, 5):
            T = texts.random_text(n, sigma, int(rng.integers(1 << 30)), sep_every=int(rng.choice([0, 50, 500])))
            with PartitionSorter(n, key_words=1) as s:
                got = gpu_sa40(torch_mod, s, T)
                stats = s.last_stats
            sa, counts = oracle_lib.prefix_doubling(T, 1)
            assert stats["active"] == counts, (n, sigma)
            assert np.array_equal(got, oracle_lib.u64_to_sa40(sa)), (n, sigma)


@TILE_ORDERS
@pytest.mark.parametrize("config", [2, 3, 4, 5])
def test_sixteen_million_symbols_pass_the_oracle_verifier(torch_mod, config, exclusive):
    """Large enough for the bucketed rank update and many radix tiles; checked with the O(n) verifier of the
    oracle (pass = byte-equal to the reference's suffix array, which is unique) and with the device verifier.
    (One K-gram word in the first sort, also for the four letters of config 4: the generations after it are what is
    looked at here; test_four_letters_start_from_keys_of_32_symbols sorts the same text the default way.)"""
    from cascade_amd import PartitionSorter, workloads, _native
    n = 1 << 24
    T = workloads.generate(config, n)
    d = to_dev(torch_mod, T)
    with PartitionSorter(n, key_words=1, device_exclusive=exclusive) as s:
        print(f"  sort config={config} n={n} exclusive={exclusive}", flush=True)
        s.set_tuning(_native.CSA_TUNE_PACK_SYMBOLS, 0)
        out = s.sort(d)
        torch_mod.cuda.synchronize()
        assert s.verify(d, out)
        got = out.cpu().numpy()
        how = s.last_stats["rank_update"]
        fused = s.last_stats["small_only"]
        dense = s.last_stats["dense"]
        stats = s.last_stats
    assert oracle_lib.is_correct_sa40(got, T)
    assert how[0] == 1  # generation 0 went through the two-pass bucketed rank update
    assert fused[0] == 0
    if config in (3, 4):  # their late generations hold small groups only (the long runs of config 5 never do)
        assert fused[-1] == 1
    if config == 4:
        # four letters: after generation 0 every suffix is still active, in 256 and then 65536 long groups. A generation
        # whose groups average more than 256 members sorts the whole partition again from rank[] and writes its ranks
        # through the bucketed update (here generation 1; generation 2 has 2^24 - 8 members in 2^16 groups, a hair below);
        # later ones, whose groups are short, change most of their ranks and take the one-pass kind of update
        active, groups = stats["active"], stats["groups"]
        want = [int(g >= 1 and 5 * active[g] >= 3 * n and active[g] > 256 * groups[g] and active[g] >= 1 << 16)
                for g in range(stats["generations"])]
        assert dense[:len(want)] == want and dense[:2] == [0, 1]
        assert all(how[g] == 1 for g in range(len(want)) if dense[g])
        assert 2 in how[1:] and 0 in how[1:]
    else:
        assert not any(dense)


@TILE_ORDERS
def test_two_dense_generations_in_a_row_on_a_four_letter_text(torch_mod, exclusive):
    """20 M symbols of four letters: generations 1 and 2 (256 and 65536 groups of far more than 256 members) both sort the
    whole partition again from the ranks read in text order; the suffix array passes the oracle's verifier and the
    generation sizes are the ones the oracle's doubling reports on a prefix-compatible smaller text (every suffix stays
    active through generation 2)."""
    from cascade_amd import PartitionSorter, workloads, _native
    n = 20_000_000
    T = workloads.generate(4, n)
    d = to_dev(torch_mod, T)
    with PartitionSorter(n, key_words=1, device_exclusive=exclusive) as s:
        print(f"  sort config=4 n={n} exclusive={exclusive}", flush=True)
        s.set_tuning(_native.CSA_TUNE_PACK_SYMBOLS, 0)
        out = s.sort(d)
        torch_mod.cuda.synchronize()
        assert s.verify(d, out)
        got = out.cpu().numpy()
        stats = s.last_stats
    assert oracle_lib.is_correct_sa40(got, T)
    assert stats["dense"][:4] == [0, 1, 1, 0] and stats["rank_update"][1] == 1 and stats["rank_update"][2] == 1
    assert stats["groups"][1] == 256 and stats["groups"][2] == 65536 and stats["active"][2] >= n - 16


@TILE_ORDERS
@pytest.mark.parametrize("key_words", [1, 4])
def test_four_letters_start_from_keys_of_32_symbols(torch_mod, key_words, exclusive):
    """The four-letter workload the default way: codes of 2 bits, 32 symbols in the key of the first sort, which stands for
    generations 0-3 of the reference's doubling with one-word keys (0-1 with four-word keys). The suffix array passes the
    oracle's verifier; the generation sizes, the covered generations' included, are those of the same text sorted from
    one K-gram word, which the oracle's doubling confirms on a text small enough for it."""
    from cascade_amd import PartitionSorter, workloads, _native
    n = 1 << 24
    T = workloads.generate(4, n)
    d = to_dev(torch_mod, T)
    with PartitionSorter(n, key_words=key_words, device_exclusive=exclusive) as s:
        print(f"  packed sort config=4 n={n} key_words={key_words} exclusive={exclusive}", flush=True)
        out = s.sort(d)
        torch_mod.cuda.synchronize()
        assert s.verify(d, out)
        got = out.cpu().numpy()
        packed = s.last_stats
        s.set_tuning(_native.CSA_TUNE_PACK_SYMBOLS, 0)
        out2 = s.sort(d)
        plain = s.last_stats
        assert torch_mod.equal(out, out2)
        small = workloads.generate(4, 1 << 17)
        s.set_tuning(_native.CSA_TUNE_PACK_SYMBOLS, 1)
        got_small = s.sort(to_dev(torch_mod, small)).cpu().numpy()
        small_stats = s.last_stats
    assert oracle_lib.is_correct_sa40(got, T)
    first = {1: 4, 4: 2}[key_words]
    assert (packed["key_symbols"], packed["first_sort_generations"]) == (32, first) and plain["first_sort_generations"] == 1
    assert packed["active"] == plain["active"] and packed["groups"][1:] == plain["groups"][1:]
    assert packed["passes"][0] == 8 and all(p == 0 for p in packed["passes"][1:first]) and not any(packed["dense"])
    sa, counts = oracle_lib.prefix_doubling(small, key_words)
    assert np.array_equal(got_small, oracle_lib.u64_to_sa40(sa)) and small_stats["active"] == counts
    assert small_stats["first_sort_generations"] == first


def test_a_dense_generation_after_one_that_was_not(torch_mod):
    """A run of 110 000 equal tokens between two stretches whose K-grams collide in some 1500 pairs: generation 1 (one long
    group, many pairs: short groups on average) gathers and leaves ranks in rank[]; the pairs dissolve, generation 2 holds
    the long group alone and sorts the whole partition again from keys of two ranks side by side (after a generation 0 or a
    dense generation it would find run ordinals there). Against the oracle, generation sizes included."""
    from cascade_amd import PartitionSorter, _native
    rng = np.random.default_rng(12)
    T = np.concatenate([rng.integers(1, 31, 25000), np.full(110000, 77), rng.integers(1, 31, 25000)]).astype(np.uint16)
    with PartitionSorter(T.size, key_words=1) as s:
        s.set_tuning(_native.CSA_TUNE_PACK_SYMBOLS, 0)
        got = s.sort(to_dev(torch_mod, T)).cpu().numpy()
        stats = s.last_stats
    sa, counts = oracle_lib.prefix_doubling(T, 1)
    assert np.array_equal(got, oracle_lib.u64_to_sa40(sa)) and stats["active"] == counts
    assert stats["dense"][:3] == [0, 0, 1], stats["dense"]


def test_generations_that_expect_their_large_groups_in_order(torch_mod):
    """A generation that follows one whose large groups were all in order leaves out the pairs of the radix sort when it
    gathers, and gathers once more with them if its own large groups turn out not to be in order. With
    CSA_TUNE_EXPECT_PRESORTED every generation starts that way: on the adversarial workload (runs and periods, whose late
    generations are in order, after early ones that are not) and on the token workload (never in order) the suffix arrays
    and the statistics must be those of the default."""
    from cascade_amd import PartitionSorter, workloads, _native
    n = 1 << 22
    for config in (5, 3):
        T = workloads.generate(config, n)
        d = to_dev(torch_mod, T)
        with PartitionSorter(n, key_words=1) as s:
            print(f"  expect-presorted config={config} n={n}", flush=True)
            out = s.sort(d)
            plain = s.last_stats
            s.set_tuning(_native.CSA_TUNE_EXPECT_PRESORTED, 1)
            out2 = s.sort(d)
            forced = s.last_stats
            assert torch_mod.equal(out, out2)
            got = out.cpu().numpy()
        assert oracle_lib.is_correct_sa40(got, T)
        for key in ("active", "groups", "big", "presorted", "passes"):
            assert plain[key] == forced[key], (config, key)
        assert any(b > 0 and p == 0 for b, p in zip(plain["big"], plain["presorted"]))  # some generation sorted its large groups
        if config == 5:
            assert any(p > 0 for p in plain["presorted"])


def test_byte_texts_start_from_keys_of_8_symbols(torch_mod):
    """A text of byte values (every value 0..255 occurs): codes of 8 bits, 8 symbols in the first key, which covers
    generations 0-1 of one-word keys. A million symbols with long repeats and a tail of zeros, against the oracle."""
    from cascade_amd import PartitionSorter
    rng = np.random.default_rng(5)
    n = 1 << 20
    T = rng.integers(0, 256, n).astype(np.uint16)
    T[n // 2:n // 2 + 50000] = T[1000:51000]
    T[n // 3:n // 3 + 3000] = 65
    T[-5:] = 0
    with PartitionSorter(n, key_words=1) as s:
        got = s.sort(to_dev(torch_mod, T)).cpu().numpy()
        stats = s.last_stats
    sa, counts = oracle_lib.prefix_doubling(T, 1)
    assert np.array_equal(got, oracle_lib.u64_to_sa40(sa)) and stats["active"] == counts
    assert (stats["key_symbols"], stats["first_sort_generations"]) == (8, 2)


def test_random_small_texts_against_the_oracle(torch_mod):
    """Many short texts over tiny alphabets (long ties, groups that straddle tiles, tails of zeros), all four key widths,
    on exact-size handles: byte-equal to the oracle's comparison sort."""
    from cascade_amd import PartitionSorter
    rng = np.random.default_rng(2024)
    for case in range(120):
        n = int(rng.integers(1, 6000))
        sigma = int(rng.integers(1, 5))
        T = rng.integers(0, sigma, n).astype(np.uint16)
        if case % 5 == 2:  # other alphabets that still pack: scattered byte values, two high bytes, up to 200 symbols
            sigma = int(rng.choice([3, 7, 16, 40, 200]))
            alphabet = rng.choice(np.arange(1, 256), size=min(sigma, 120), replace=False).astype(np.uint16)
            if case % 10 == 2:
                alphabet = np.concatenate([alphabet[:sigma // 2 + 1], alphabet[:sigma // 2 + 1] + 0x0700]).astype(np.uint16)
            T = alphabet[rng.integers(0, alphabet.size, n)]
        if case % 3 == 0:
            T[-int(rng.integers(1, min(n, 40) + 1)):] = 0
        if case % 4 == 1 and n > 600:
            T[n // 2:n // 2 + 256] = T[:256]  # a long repeat
        kw = 1 + case % 4
        with PartitionSorter(n, key_words=kw) as s:
            print(f"  random case={case} n={n} sigma={sigma} key_words={kw}", flush=True)
            got = s.sort(to_dev(torch_mod, T)).cpu().numpy()
        assert np.array_equal(got, oracle_lib.build_sa40(T)), (case, n, sigma, kw)


def test_random_alphabets_structures_and_paths_against_the_oracle(torch_mod):
    """600 random texts: alphabets that pack into 1, 2, 4 or 8 bits, that pack through their byte ranks, that do not pack;
    repeats, runs, periodic stretches and zero tails laid over them; all four key widths; and, at random, the knobs that
    force the other paths (one K-gram word in the first sort, every generation expecting its large groups in order, the
    bucketed rank updates). Suffix array and generation sizes against the oracle's doubling. (A run of this generator over
    some 350 000 texts found the one dense-after-gather case that test_a_dense_generation_after_one_that_was_not pins.)"""
    from cascade_amd import PartitionSorter, _native
    rng = np.random.default_rng(31)
    for case in range(600):
        n = max(1, int(rng.choice([1, 2, 3, 5, 17, 63, 64, 65, 255, 1000, 4097, 20000])) + int(rng.integers(-3, 4)))
        kind = int(rng.integers(0, 7))
        if kind == 0:
            alphabet = np.arange(int(rng.integers(1, 5)))
        elif kind == 1:
            alphabet = rng.choice(np.arange(0, 256), size=int(rng.integers(1, 200)), replace=False)
        elif kind == 2:
            lo = rng.choice(np.arange(0, 256), size=int(rng.integers(1, 12)), replace=False)
            hi = rng.choice(np.arange(0, 256), size=int(rng.integers(1, 12)), replace=False)
            alphabet = (hi[:, None] * 256 + lo[None, :]).ravel()
        elif kind == 3:
            alphabet = rng.choice(np.arange(0, 65536), size=int(rng.integers(2, 3000)), replace=False)
        elif kind == 4:
            alphabet = np.array([65, 67, 71, 84])
        elif kind == 5:
            alphabet = np.array([int(rng.integers(0, 65536))])
        else:
            alphabet = np.arange(256)
        T = alphabet.astype(np.uint16)[rng.integers(0, alphabet.size, n)]
        for _ in range(int(rng.integers(0, 4))):
            if n < 8:
                break
            a, length = int(rng.integers(0, n - 4)), int(rng.integers(1, max(2, n // 3)))
            what = int(rng.integers(0, 4))
            if what == 0:
                b = int(rng.integers(0, n - 4))
                length = min(length, n - max(a, b))
                T[b:b + length] = T[a:a + length].copy()
            elif what == 1:
                T[a:a + length] = T[a]
            elif what == 2:
                length = min(length, n - a)
                T[a:a + length] = np.resize(T[a:a + int(rng.integers(2, 9))].copy(), length)
            else:
                T[-min(n, int(rng.integers(1, 70))):] = 0
        kw = int(rng.integers(1, 5))
        knobs = [int(rng.integers(0, 3)) == 0 for _ in range(3)]
        with PartitionSorter(n, key_words=kw) as s:
            if knobs[0]:
                s.set_tuning(_native.CSA_TUNE_PACK_SYMBOLS, 0)
            if knobs[1]:
                s.set_tuning(_native.CSA_TUNE_EXPECT_PRESORTED, 1)
            if knobs[2]:
                s.set_tuning(_native.CSA_TUNE_DEFER_MIN, 1)
                s.set_tuning(_native.CSA_TUNE_WINDOW_MIN_CHANGED, 1)
            if case % 100 == 0:
                print(f"  random text case={case} n={n} alphabet kind={kind} key_words={kw} knobs={knobs}", flush=True)
            got = s.sort(to_dev(torch_mod, T)).cpu().numpy()
            stats = s.last_stats
        sa, counts = oracle_lib.prefix_doubling(T, kw)
        assert np.array_equal(got, oracle_lib.u64_to_sa40(sa)) and stats["active"] == counts, (case, n, kind, kw, knobs)


def test_bucketed_rank_updates_at_small_and_ragged_sizes(torch_mod):
    """The bucketed rank updates normally serve lists of millions of suffixes: generation 0 sends (position, rank)
    records through value-less radix passes and a window placement, later generations (position, rank) pairs through one
    pass and a windowed scatter. With their thresholds at 1 (csa_set_tuning) every list takes them: sizes
    around the tile, window and pass boundaries, checked against the oracle, and the library must report that it went
    that way."""
    from cascade_amd import PartitionSorter, workloads, _native
    rng = np.random.default_rng(77)
    sizes = [1, 2, 5, 255, 1024, 1025, 8191, 8193, (1 << 14) - 1, 1 << 14, (1 << 14) + 1, 16385 * 3, (1 << 16) + 7,
             (1 << 18) - 3, (1 << 20) + 11]
    for case, n in enumerate(sizes):
        if case % 3 == 0:
            T = workloads.generate(3, n) if n >= 64 else rng.integers(0, 3, n).astype(np.uint16)
        elif case % 3 == 1:
            T = rng.integers(0, 4, n).astype(np.uint16)
        else:
            T = workloads.generate(5, n) if n >= 64 else np.zeros(n, dtype=np.uint16)
        with PartitionSorter(n, key_words=1 + case % 2) as s:
            print(f"  bucketed case={case} n={n} key_words={s.key_words}", flush=True)
            s.set_tuning(_native.CSA_TUNE_DEFER_MIN, 1)
            s.set_tuning(_native.CSA_TUNE_WINDOW_MIN_CHANGED, 1)
            got = s.sort(to_dev(torch_mod, T)).cpu().numpy()
            how = s.last_stats["rank_update"]
        if n <= 1 << 16:
            assert np.array_equal(got, oracle_lib.build_sa40(T)), (case, n)
        else:  # the oracle's O(n) verifier: pass = byte-equal to the one correct suffix array
            assert oracle_lib.is_correct_sa40(got, T), (case, n)
        assert how[0] == 1, (case, n, how)


@pytest.mark.parametrize("key_words", [3, 4])
def test_keys_of_three_and_four_words_on_deep_repeats(torch_mod, key_words):
    """The reference's default key is 4 words (include/Packed_Prefix.hpp:20-24): the same suffix array, fewer and
    smaller generations, whose sizes must be the oracle's for that key width."""
    from cascade_amd import PartitionSorter, workloads
    with PartitionSorter(1 << 19, key_words=key_words) as s:
        for config in (3, 5, 4):
            T = workloads.generate(config, 1 << 19)
            got = gpu_sa40(torch_mod, s, T)
            sa, counts = oracle_lib.prefix_doubling(T, key_words)
            assert np.array_equal(got, oracle_lib.u64_to_sa40(sa)), config
            assert s.last_stats["active"] == counts, config
            assert s.last_stats["passes"][0] >= 1


def test_three_dispatcher_threads_with_their_own_handles_and_streams(torch_mod):
    """The reference drives three buffer sets from three threads, one stream each (include/GPU_SACA.hpp:90-91,
    src/GPU_SACA.cu:1539-1589): handles must not share state. Three threads sort different partitions at once,
    several times over, each on its own stream and handle; every result is byte-equal to the oracle's."""
    import threading
    from cascade_amd import PartitionSorter
    torch = torch_mod
    rng = np.random.default_rng(33)
    jobs = []
    for k in range(3):
        texts_k = [texts.random_text(int(rng.integers(20000, 90000)), 2 + k, 100 * k + r, sep_every=0) for r in range(4)]
        jobs.append([(T, oracle_lib.build_sa40(T)) for T in texts_k])
    errors = []

    def worker(k):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream), PartitionSorter(100000, key_words=1 + k % 2) as s:
                for rep in range(3):
                    for T, want in jobs[k]:
                        d = torch.from_numpy(np.ascontiguousarray(T).view(np.int16)).cuda(non_blocking=False)
                        got = s.sort(d)
                        stream.synchronize()
                        if not np.array_equal(got.cpu().numpy(), want):
                            errors.append((k, rep, T.size))
        except Exception as e:  # noqa: BLE001 - reported below, in the main thread
            errors.append((k, repr(e)))

    print("  three threads, three handles, three streams", flush=True)
    threads = [threading.Thread(target=worker, args=(k,)) for k in range(3)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


@pytest.mark.parametrize("config,key_words", [(3, 1), (3, 4), (2, 2), (4, 1)])
def test_generation_sizes_are_those_the_references_own_predictor_gives(torch_mod, tmp_path, config, key_words):
    """src/sa_structure.cpp of the reference (compiled from its one source file into oracle/_ref) predicts, from a finished
    suffix array, how many suffixes retire at every generation of a run, and verifies the array while it reads it. Two
    million symbols of the token workloads and of the four-letter workload (whose first sort takes keys of 32 packed
    symbols and stands for several generations): the sizes the library reports for every generation, the covered ones
    included, must be the predictor's, and its file must pass the tool's own order and permutation checks."""
    from cascade_amd import PartitionSorter, workloads
    if not os.path.exists(oracle_lib.SA_STRUCTURE):
        pytest.skip("oracle/_ref/sa_structure is not built (make -C oracle where the reference tree is present)")
    n = 1 << 21
    T = workloads.generate(config, n)
    with PartitionSorter(n, key_words=key_words) as s:
        print(f"  sort against sa_structure config={config} key_words={key_words}", flush=True)
        got = s.sort(to_dev(torch_mod, T)).cpu().numpy()
        stats = s.last_stats
    ell = 4 * key_words
    theirs = oracle_lib.reference_structure(T, got, ell, ell, [n], tmp_path)
    assert oracle_lib.active_sizes_from_retirements(n, theirs["retire_hist"]) == stats["active"], (stats["active"], theirs["retire_hist"])


def test_the_references_own_tool_accepts_the_command_line_builders_file(tmp_path):
    """tools/sa_convert.cpp of the reference, compiled from its one source file into oracle/_ref (oracle/Makefile), is
    what the reference runs on a finished 40-bit suffix array: the file cascade_sa writes passes its size checks and
    its spot check of the order (100 000 adjacent pairs, the reference's comparator), gets an index.meta, and widens,
    through the reference's own sa40 loader, to the oracle's 64-bit array."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    tool, exe = os.path.join(root, "oracle", "_ref", "sa_convert"), os.path.join(root, "cascade_amd", "cascade_sa")
    if not os.path.exists(tool):
        pytest.skip("oracle/_ref/sa_convert is not built (make -C oracle where the reference tree is present)")
    T = texts.random_text(300000, 50257, 8, sep_every=900)
    T[200000:260000] = T[1000:61000]
    ip, op = tmp_path / "t.u16", tmp_path / "t.sa40"
    T.astype("<u2").tofile(ip)
    r = subprocess.run([exe, str(ip), str(op)], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([tool, "--meta-only", "--sa", str(op), "--text", str(ip), "--sym-bytes", "2", "--index-dir", str(tmp_path / "index")],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and "spot-check passed" in r.stderr and (tmp_path / "index" / "index.meta").exists(), r.stderr
    r = subprocess.run([tool, "--widen", "--in", str(op), "--out", str(tmp_path / "t.u64")], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.fromfile(tmp_path / "t.u64", dtype="<u8"), oracle_lib.sa40_to_u64(oracle_lib.build_sa40(T)))


def test_command_line_builder_writes_the_oracles_suffix_array(tmp_path):
    """cascade_amd/cascade_sa <text-file> <suffix-array-file>: the reference's program (src/main.cu:12-46) through the
    C++ mirror of its builder class; the file it writes is the oracle's, byte for byte; a missing input ends it with
    an error message and status 1, as the reference's error policy does."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cascade_amd", "cascade_sa")
    for name, T in (("c1", texts.random_text(200000, 50257, 1, sep_every=1000)), ("ties", texts.random_text(50000, 2, 2, sep_every=0)),
                    ("empty", np.zeros(0, dtype=np.uint16))):
        ip, op = tmp_path / f"{name}.u16", tmp_path / f"{name}.sa40"
        T.astype("<u2").tofile(ip)
        print(f"  cascade_sa {name} n={T.size}", flush=True)
        for key_words in (1, 4):
            r = subprocess.run([exe, str(ip), str(op), str(key_words)], capture_output=True, text=True, timeout=100)
            assert r.returncode == 0 and "Time taken" in r.stderr, r.stderr
            assert np.array_equal(np.fromfile(op, dtype=np.uint8), oracle_lib.build_sa40(T)), (name, key_words)
    r = subprocess.run([exe, str(tmp_path / "missing.u16"), str(tmp_path / "x.sa40")], capture_output=True, text=True, timeout=100)
    assert r.returncode == 1 and "cannot open" in r.stderr

