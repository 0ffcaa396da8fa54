"""The kernel sources of cascade_amd/csrc, compiled for the CPU against tests/cpu_emu (a stand-in for the HIP
runtime and the wave64 intrinsics), must reproduce the oracle's suffix arrays. This checks the kernels' logic
and indexing where no GPU exists; the library built here is test infrastructure and is never loaded by the
product. Small inputs only: every wave operation is a thread barrier on the CPU."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

import oracle_lib
import texts
from cascade_amd import _native

EMU_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpu_emu")


def load_emulation(target):
    subprocess.run(["make", "-C", EMU_DIR, target], check=True, capture_output=True)
    lib = C.CDLL(os.path.join(EMU_DIR, target))
    vp, u64, u32, i32 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_int
    lib.csa_create.argtypes = [u64, i32, C.POINTER(vp)]
    lib.csa_destroy.argtypes = [vp]
    lib.csa_sort_partition_u16_dev.argtypes = [vp, vp, u64, u64, vp, vp, u32, C.POINTER(_native.CsaStats)]
    lib.csa_radix_sort_pairs_dev.argtypes = [vp, vp, vp, u64, i32, i32, vp]
    lib.csa_last_error.restype = C.c_char_p
    lib.csa_partition_ids_u16_dev.argtypes = [vp, u64, u64, vp, i32, u32, vp, vp, vp, vp]
    lib.csa_stage_slab_u16_dev.argtypes = [vp, u64, vp, u64, i32, vp, u32, u64, i32, vp, vp, vp]
    lib.csa_scatter_to_rank_order_dev.argtypes = [vp, vp, vp, u64, vp, vp]
    lib.csa_count_messages_dev.argtypes = [vp, vp, vp, u64, u64, i32, u32, vp, vp]
    lib.csa_message_offsets_dev.argtypes = [vp, u32, vp]
    lib.csa_emit_messages_dev.argtypes = [vp, vp, vp, u64, u64, i32, vp, u32, vp, vp, vp, vp]
    lib.csa_join_messages_dev.argtypes = [vp, vp, u32, vp, vp, vp, u64, vp]
    lib.csa_join_messages_sorted_dev.argtypes = [vp, vp, vp, u32, vp, vp, vp, u64, vp]
    lib.csa_sort_init_dev.argtypes = [vp, vp, i32, vp, vp, u64, u32, vp, vp, vp, vp, vp, vp, vp]
    lib.csa_sort_rerank_dev.argtypes = [vp, vp, vp, vp, u64, vp, vp, u32, u64, u32, vp, vp, vp, vp, vp, vp, vp]
    lib.csa_sort_init_slabs.argtypes = [vp, C.POINTER(_native.CsaSlab), u32, u64, i32, u32, u64, vp, vp, vp]
    lib.csa_sort_rerank_slabs.argtypes = [vp, C.POINTER(_native.CsaSlab), u32, u64, u64, u64, u32, u64, vp, vp, vp]
    lib.csa_scatter_slabs.argtypes = [vp, C.POINTER(_native.CsaSlab), u32, u64, u64, u64, vp]
    lib.csa_create_steps.argtypes = [u64, i32, C.POINTER(vp)]
    lib.csa_step_bytes_per_suffix.restype = u64
    lib.csa_step_bytes_per_suffix.argtypes = [i32]
    lib.csa_workspace_bytes.restype = u64
    lib.csa_workspace_bytes.argtypes = [u64]
    lib.csa_scratch_high_water.restype = u64
    lib.csa_scratch_high_water.argtypes = [vp]
    lib.csa_last_step_result.argtypes = [vp, C.POINTER(_native.CsaStepResult)]
    lib.csa_set_tuning.argtypes = [vp, i32, u32]
    return lib


@pytest.fixture(scope="module")
def emu():
    """The kernels with small tiles and low thresholds, so that texts of a few thousand symbols reach every path."""
    return load_emulation("libcascade_emu.so")


@pytest.fixture(scope="module")
def emu_dev():
    """The kernels with the tile sizes and thresholds of the device build."""
    return load_emulation("libcascade_emu_dev.so")


def steps_handle(lib, key_words):
    """For multi_partition.build_sa: a handle of exactly the largest partition's capacity, made for the steps."""
    def make(max_part_sz):
        h = C.c_void_p()
        assert lib.csa_create_steps(max_part_sz, key_words, C.byref(h)) == 0, lib.csa_last_error()
        return h
    return make


def emu_sort(lib, T, key_words, pack=True, expect_presorted=False):
    """pack=False: the first sort takes one K-gram word even when the alphabet is small (CSA_TUNE_PACK_SYMBOLS 0), for the
    tests that aim at what the generations after it do on such texts. expect_presorted: CSA_TUNE_EXPECT_PRESORTED 1."""
    T = np.ascontiguousarray(T, dtype=np.uint16)
    n = T.size
    h = C.c_void_p()
    assert lib.csa_create(max(n, 1), key_words, C.byref(h)) == 0
    if not pack:
        assert lib.csa_set_tuning(h, _native.CSA_TUNE_PACK_SYMBOLS, 0) == 0
    if expect_presorted:
        assert lib.csa_set_tuning(h, _native.CSA_TUNE_EXPECT_PRESORTED, 1) == 0
    out = np.zeros(5 * n + 8, dtype=np.uint8)
    st = _native.CsaStats()
    rc = lib.csa_sort_partition_u16_dev(h, T.ctypes.data, n, 0, out.ctypes.data, None, 0, C.byref(st))
    lib.csa_destroy(h)
    assert rc == 0, lib.csa_last_error()
    emu_sort.rank_update = [int(st.rank_update[i]) for i in range(st.generations)]
    emu_sort.small_only = [int(st.small_only[i]) for i in range(st.generations)]
    emu_sort.dense = [int(st.dense[i]) for i in range(st.generations)]
    emu_sort.presorted = [int(st.presorted[i]) for i in range(st.generations)]
    emu_sort.key_symbols, emu_sort.first_sort_generations = int(st.key_symbols), int(st.first_sort_generations)
    emu_sort.passes = [int(st.passes[i]) for i in range(st.generations)]
    return out[:5 * n], [int(st.active[i]) for i in range(st.generations)], [int(st.big[i]) for i in range(st.generations)]


CASES = ["rand_n17_s2", "rand_n1000_s2", "rand_n1000_s65536", "hand_1", "hand_15", "hand_18", "hand_23"]


@pytest.mark.parametrize("key_words", [1, 2])
def test_fixtures_through_the_emulated_kernels(emu, key_words):
    suite = dict(texts.fixture_suite())
    for name in CASES:
        T = suite[name]
        got, active, _ = emu_sort(emu, T, key_words)
        assert np.array_equal(got, oracle_lib.build_sa40(T)), name
        _, counts = oracle_lib.prefix_doubling(T, key_words)
        assert active == counts, name


@pytest.mark.parametrize("n,sigma,key_words,pack", [(70000, 3, 1, True), (50000, 300, 1, False), (40000, 2, 2, False)])
def test_the_device_builds_tile_sizes_in_the_emulation(emu_dev, n, sigma, key_words, pack):
    """The same sources compiled with the device build's own constants (1024-thread workgroups, tiles of 16384 pairs, 2048
    members per small-group tile): texts of several tiles with a long repeat and a zero tail."""
    T = texts.random_text(n, sigma, n + sigma, sep_every=0)
    T[n // 3:n // 3 + n // 5] = T[:n // 5]
    T[-9:] = 0
    got, active, _ = emu_sort(emu_dev, T, key_words, pack=pack)
    assert np.array_equal(got, oracle_lib.build_sa40(T))
    _, counts = oracle_lib.prefix_doubling(T, key_words)
    assert active == counts


def test_a_pipeline_at_the_device_builds_tile_sizes(emu_dev):
    """Partition ids, slab staging, the two partition steps with their messages and the final scatter at the device build's
    tile sizes: 30000 suffixes in 5 partitions."""
    import multi_partition
    T = texts.random_text(30000, 4, 5, sep_every=0)
    T[12000:17000] = T[1000:6000]
    T[-6:] = 0
    sa, gens = multi_partition.build_sa(emu_dev, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a, T, 5, key_words=1,
                                        step_handle=steps_handle(emu_dev, 1))
    want, _ = oracle_lib.prefix_doubling(T, 1)
    assert np.array_equal(sa, want) and gens >= 5


@pytest.mark.parametrize("switch", ["HIPEMU_REVERSE", "HIPEMU_LANES_REVERSE"])
def test_results_do_not_depend_on_the_order_of_workgroups_and_lanes(switch):
    """The emulation runs the workgroups of a launch one after the other, by blockIdx, and the lanes of a workgroup as fibers
    that hand over to the next lane at a barrier. HIPEMU_REVERSE=1 runs the workgroups from the last to the first: tiles
    numbered by arrival, look-back chains and atomically reserved ranges must give the same results. HIPEMU_LANES_REVERSE=1
    hands over to the lane before instead: a value that one lane writes and another reads between two barriers, without an
    order of their own, would show under one of the two directions. (Process-wide switches, hence a process of its own.)"""
    import sys
    env = dict(os.environ, **{switch: "1"})
    chosen = ("fixtures_through or random_texts_through or random_pipelines_through or emulated_message_kernels or partition_ids_match "
              "or slab_staging or three_and_four_words")
    run = subprocess.run([sys.executable, "-m", "pytest", os.path.abspath(__file__), "-x", "-q", "-k", chosen], env=env, capture_output=True, text=True)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-2000:]


def test_random_texts_through_the_emulated_sort(emu):
    """Random alphabets (1 to 65536 symbols), structures (plain, a long repeat, a zero tail, a run of one symbol, a period),
    key widths and tuning knobs (packed first sort on and off, the speculative gather): the suffix array and every
    generation's active-set size are the oracle's."""
    rng = np.random.default_rng(77)
    for case in range(60):
        n = int(rng.integers(1, 3000))
        sigma = int(rng.choice([1, 2, 3, 4, 7, 16, 200, 300, 65536]))
        T = rng.integers(0, sigma, n).astype(np.uint16)
        shape = int(rng.integers(0, 5))
        if shape == 1 and n > 100:
            length = int(rng.integers(10, n // 2))
            T[n - length:] = T[:length]
        if shape == 2:
            T[-int(rng.integers(1, 40)):] = 0
        if shape == 3 and n > 100:
            a = int(rng.integers(0, n // 2))
            T[a:a + int(rng.integers(5, n // 2))] = T[a]
        if shape == 4 and n > 100:
            period = int(rng.integers(1, 9))
            a = int(rng.integers(0, n // 2))
            stretch = int(rng.integers(20, n // 2))
            T[a:a + stretch] = np.resize(T[a:a + period], stretch)
        key_words = int(rng.integers(1, 5))
        pack, speculate = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        got, active, _ = emu_sort(emu, T, key_words, pack=pack, expect_presorted=speculate)
        assert np.array_equal(got, oracle_lib.build_sa40(T)), (case, n, sigma, shape, key_words, pack, speculate)
        _, counts = oracle_lib.prefix_doubling(T, key_words)
        assert active == counts, (case, n, sigma, shape, key_words, pack, speculate)


@pytest.mark.parametrize("key_words", [3, 4])
def test_keys_of_three_and_four_words(emu, key_words):
    # wide keys (four words, 16 symbols, are the reference's default) run as one-word keys whose first generations stand
    # for generation 0: 4 -> 8 -> 16 symbols, or 4 -> 8 -> 12 with a second step that looks only 4 symbols ahead. The
    # generation sizes must be the oracle's for that key width; texts shorter than a key, and runs that tie over a whole
    # key, are the edge cases
    suite = dict(texts.fixture_suite())
    for name, T in [(n_, suite[n_]) for n_ in ("rand_n17_s2", "rand_n1000_s2", "hand_15")] + [
            ("run", np.concatenate([np.full(40, 3, dtype=np.uint16), texts.random_text(300, 2, 9, sep_every=0)])),
            ("short", np.array([2, 1, 2, 1, 2], dtype=np.uint16))]:
        got, active, _ = emu_sort(emu, T, key_words)
        assert np.array_equal(got, oracle_lib.build_sa40(T)), name
        _, counts = oracle_lib.prefix_doubling(T, key_words)
        assert active == counts, name


@pytest.mark.parametrize("key_words", [1, 2])
def test_text_at_every_alignment_inside_an_eight_byte_word(emu, key_words):
    # the first pass stages the text with aligned 8-byte loads: the text may start anywhere inside such a word, and
    # its end (here a run of zeros, which ties with the key padding) anywhere too
    rng = np.random.default_rng(7)
    backing = np.zeros(1400, dtype=np.uint16)
    base_off = (-backing.ctypes.data // 2) % 4  # symbols to the next 8-byte boundary
    for off in range(4):
        for n in ((641 + off, 644) if key_words == 1 else (643 - off,)):
            T = backing[base_off + off:base_off + off + n]
            T[:] = rng.integers(0, 3, n)
            T[-5:] = 0
            assert (T.ctypes.data % 8) == 2 * off
            got, _, _ = emu_sort(emu, T, key_words)
            assert np.array_equal(got, oracle_lib.build_sa40(np.array(T))), (off, n)


@pytest.mark.parametrize("after_run", [2, 9])
def test_large_groups_that_are_in_order_already_skip_the_sort(emu, after_run):
    # A run of one token and a periodic stretch: from the second generation on, the gathered ranks of every large group
    # rise or fall along the list (falling in the run when a smaller symbol follows it, rising when a larger one does),
    # so the generation ranks them where they stand instead of sorting them. Random text around them keeps small groups
    # in the same lists; the two-letter stretch gives generation 1 large groups that are out of order, which it sorts.
    T = np.concatenate([texts.random_text(1300, 2, 21, sep_every=0) + 6, np.full(700, 5, dtype=np.uint16),
                        np.array([after_run], dtype=np.uint16), np.tile(np.array([3, 1, 4, 1, 5, 9, 2], dtype=np.uint16), 150),
                        texts.random_text(400, 3, 22, sep_every=0)])
    got, active, big = emu_sort(emu, T, 1, pack=False)
    assert np.array_equal(got, oracle_lib.build_sa40(T))
    _, counts = oracle_lib.prefix_doubling(T, 1)
    assert active == counts
    presorted = emu_sort.presorted
    assert any(p > 0 for p in presorted), (big, presorted)
    assert all(p in (0, b) for p, b in zip(presorted, big))        # all of a generation's large groups, or none
    assert any(b > 0 and p == 0 for p, b in zip(presorted, big))   # and some generation did sort its large groups
    # A generation that follows one whose large groups were all in order gathers without the pairs of the radix sort, and
    # once more with them if its own large groups are not in order: with every generation starting that way, the ones that
    # do sort take the second gather, and nothing else changes
    got2, active2, big2 = emu_sort(emu, T, 1, pack=False, expect_presorted=True)
    assert np.array_equal(got2, got) and (active2, big2, emu_sort.presorted) == (active, big, presorted)


def test_small_and_large_groups_take_both_paths(emu):
    # 2 symbols, no separators: generation 1 has a few huge groups (radix path), later ones small groups (in-tile path)
    T = texts.random_text(6000, 2, 5, sep_every=0)
    got, active, big = emu_sort(emu, T, 1, pack=False)
    assert np.array_equal(got, oracle_lib.build_sa40(T))
    assert big[1] > 0 and any(b == 0 and a > 0 for a, b in zip(active[2:], big[2:]))
    # generation 0 takes the bucketed rank update here (records through one value-less radix pass on 4 position bits,
    # then windows of 512 ranks) and later ones the one-pass kind (the emulation library is built with tiny thresholds
    # and windows for both); the short fixtures above write their ranks directly
    assert emu_sort.rank_update[0] == 1 and 2 in emu_sort.rank_update[1:]
    # once a generation had no large group, the following ones run as the fused small-group generation
    first_small = big.index(0, 1)
    assert emu_sort.small_only == [0] * (first_small + 1) + [1] * (len(big) - first_small - 1) and 1 in emu_sort.small_only


@pytest.mark.parametrize("name,key_words", [("one_symbol", 1), ("period_3", 4)])
def test_dense_generations_sort_the_whole_partition_again(emu, name, key_words):
    """Texts whose suffixes nearly all stay tied, in a handful of long groups, for many generations: those generations take
    the dense form (keys (rank[x], rank[x + h]) read in text order, every suffix sorted again, ranks back through the
    bucketed update). Same suffix array and the same active counts as the oracle's doubling, for plain and folded wide keys."""
    T = {"one_symbol": np.full(1700, 7, dtype=np.uint16), "period_3": np.tile(np.array([3, 1, 4], dtype=np.uint16), 560)}[name]
    got, active, _ = emu_sort(emu, T, key_words, pack=False)
    sa, counts = oracle_lib.prefix_doubling(T, key_words)
    assert np.array_equal(got, oracle_lib.u64_to_sa40(sa)) and active == counts
    assert emu_sort.dense[0] == 0 and sum(emu_sort.dense) >= 5 and emu_sort.dense[-1] == 0
    assert all(u == 1 for u, d in zip(emu_sort.rank_update, emu_sort.dense) if d)


def test_a_dense_generation_after_one_that_was_not(emu):
    """A long run of one token and a stretch whose K-grams collide in pairs: generation 1 holds the run's one long group and
    a couple of hundred pairs (short groups on average: the gather form, which leaves ranks in rank[]); the pairs dissolve
    there, and generation 2 is left with the long group alone and takes the dense form, on keys of two ranks side by side
    (a generation 0 or a dense generation before it would have left run ordinals instead)."""
    rng = np.random.default_rng(3)
    T = np.concatenate([rng.integers(1, 7, 350), np.full(1400, 9), rng.integers(1, 7, 350)]).astype(np.uint16)
    got, active, _ = emu_sort(emu, T, 1, pack=False)
    sa, counts = oracle_lib.prefix_doubling(T, 1)
    assert np.array_equal(got, oracle_lib.u64_to_sa40(sa)) and active == counts
    assert emu_sort.dense[:3] == [0, 0, 1], emu_sort.dense


PACKED_CASES = {
    "four_letters": (np.arange(4), 1, 32, 4),                    # codes of 2 bits
    "one_letter": (np.array([7]), 1, 64, 5),                     # with the padding's zero: 2 codes, 1 bit
    "acgt_ascii": (np.array([65, 67, 71, 84]), 1, 16, 3),        # 5 low-byte values with zero: 4 bits
    "bytes": (np.arange(256), 1, 8, 2),
    "bytes_two_words": (np.arange(256), 2, 8, 1),                # the caller's own key width, in one word
    "high_bytes": (np.array([0x0101, 0x0102, 0x0201]), 1, 16, 3),  # 3 x 3 byte ranks: 9 codes
    "three_words": (np.array([1, 2, 3]), 3, 24, 2),              # 12 -> 24 symbols of 2 bits; 48 would not fit
    "four_words": (np.arange(4), 4, 32, 2),
    "bytes_three_words": (np.arange(256), 3, 4, 1),              # 12 bytes do not fit a key: one K-gram word, as ever
    "large_alphabet": (np.arange(1000, 1300), 1, 4, 1),
}


@pytest.mark.parametrize("name", sorted(PACKED_CASES))
def test_small_alphabets_start_from_keys_of_many_symbols(emu, name):
    """A text of at most 256 different symbols (by the values its low and high bytes take, zero, the key padding,
    counted in) is sorted first on keys of as many packed symbols as 64 bits hold: codes of 1, 2, 4 or 8 bits, 4 W 2^j
    symbols. That sort stands for the first 1 + j generations of the oracle's doubling: the suffix array is the oracle's, and
    so is every generation's active count, those of the covered generations included (counted on prefixes of the sorted
    keys). The texts hold a long repeat that keeps suffixes tied past the key, and zeros at the end, which tie with the
    padding of the last keys."""
    alphabet, key_words, key_symbols, first = PACKED_CASES[name]
    rng = np.random.default_rng(len(name))
    body = alphabet[rng.integers(0, alphabet.size, 900 if name == "one_letter" else 2500)].astype(np.uint16)  # (one letter: every generation is dense)
    T = np.concatenate([body, body[300:900], body[:50], np.zeros(3, dtype=np.uint16)]).astype(np.uint16)
    got, active, _ = emu_sort(emu, T, key_words)
    sa, counts = oracle_lib.prefix_doubling(T, key_words)
    assert np.array_equal(got, oracle_lib.u64_to_sa40(sa))
    assert active == counts
    assert (emu_sort.key_symbols, emu_sort.first_sort_generations) == (key_symbols, first)
    assert all(p == 0 for p in emu_sort.passes[1:first])
    if first > 1 or name == "bytes_two_words":
        # the same text without the packed keys: the same array, the same counts
        got2, active2, _ = emu_sort(emu, T, key_words, pack=False)
        assert np.array_equal(got2, got) and active2 == counts and emu_sort.first_sort_generations == 1


def test_emulated_radix_sort_matches_stable_sort(emu):
    rng = np.random.default_rng(1)
    n = 5000
    keys = rng.integers(0, 1 << 40, n).astype(np.uint64)
    vals = np.arange(n, dtype=np.uint32)
    wk, wv = oracle_lib.stable_sort_pairs(keys, vals, 3, 37)
    h = C.c_void_p()
    assert emu.csa_create(n, 1, C.byref(h)) == 0
    k, v = keys.copy(), vals.copy()
    assert emu.csa_radix_sort_pairs_dev(h, k.ctypes.data, v.ctypes.data, n, 3, 37, None) == 0
    emu.csa_destroy(h)
    assert np.array_equal(k, wk) and np.array_equal(v, wv)


def test_emulated_radix_sort_without_allocation_matches_the_one_with_a_handle(emu):
    """csa_radix_sort_pairs_static_dev (fixed scratch inside the library, which keeps the last call's contents): two
    calls in a row, the second smaller and over another bit range, each equal to csa_radix_sort_pairs_dev and to the
    oracle's stable sort; sizes beyond the fixed scratch are refused."""
    emu.csa_radix_sort_pairs_static_dev.restype = C.c_int
    emu.csa_radix_sort_pairs_static_dev.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_void_p]
    rng = np.random.default_rng(4)
    h = C.c_void_p()
    assert emu.csa_create(20000, 1, C.byref(h)) == 0
    for n, b, e in ((9000, 0, 40), (3001, 5, 29), (1, 0, 64), (1024, 8, 24)):
        keys = rng.integers(0, 1 << 63, n).astype(np.uint64) >> np.uint64(rng.integers(0, 40))
        vals = rng.permutation(n).astype(np.uint32)
        k0, v0 = keys.copy(), vals.copy()
        assert emu.csa_radix_sort_pairs_dev(h, k0.ctypes.data, v0.ctypes.data, n, b, e, None) == 0
        k1, v1 = keys.copy(), vals.copy()
        assert emu.csa_radix_sort_pairs_static_dev(k1.ctypes.data, v1.ctypes.data, n, b, e, None) == 0
        wk, wv = oracle_lib.stable_sort_pairs(keys, vals, b, e)
        assert np.array_equal(k1, k0) and np.array_equal(v1, v0), (n, b, e)
        assert np.array_equal(k1, wk) and np.array_equal(v1, wv), (n, b, e)
    emu.csa_destroy(h)
    big = np.zeros(20001, dtype=np.uint64)
    assert emu.csa_radix_sort_pairs_static_dev(big.ctypes.data, big.ctypes.data, 20001, 0, 64, None) == -2


@pytest.mark.parametrize("words,p", [(1, 1), (1, 3), (2, 2), (2, 16), (2, 17), (2, 256), (3, 300), (4, 5), (4, 64)])
def test_emulated_partition_ids_match_the_oracle(emu, words, p):
    """Pivot counts that fill the searched table exactly (p = 2^k) and that leave it padded; texts over three symbols, of one
    symbol and of separators only (all-ones K-grams, the value the table's padding holds): most suffixes start like some
    pivot there and are placed by the search over all key words."""
    rng = np.random.default_rng(words * 1000 + p)
    for n in (1, 64, 65, 2049, 4500, 3001, 3002):
        T = texts.random_text(n, 3, n + p, sep_every=0)
        if n == 3001:
            T[:] = 7
            T[n // 2] = 8
        if n == 3002:
            T[:] = 0xFFFF
            T[n // 3] = 5
        pivots = oracle_lib.sample_pivots(T, p, words, rng, duplicates=True)
        bits = oracle_lib.partition_id_bits(p)
        ids = np.zeros(n, dtype=np.uint16)
        packed = np.zeros(((n + 63) // 64) * bits + 1, dtype=np.uint64)
        sizes = np.zeros(p, dtype=np.uint64)
        rc = emu.csa_partition_ids_u16_dev(T.ctypes.data, n, n, pivots.ctypes.data if p > 1 else None, words, p, ids.ctypes.data,
                                           packed.ctypes.data, sizes.ctypes.data, None)
        assert rc == 0, emu.csa_last_error()
        want_ids, want_sizes = oracle_lib.partition_ids(T, pivots, p, words)
        assert np.array_equal(ids, want_ids) and np.array_equal(sizes, want_sizes), n
        nw = oracle_lib.packed_words(n, bits)
        assert np.array_equal(packed[:nw], oracle_lib.pack_partition_ids(want_ids, bits)[:nw]) and not packed[nw:].any(), n


@pytest.mark.parametrize("generation0,ctx,key_words", [(True, 4, 1), (False, 16, 2)])
def test_emulated_slab_staging_and_rank_order_scatter(emu, generation0, ctx, key_words):
    rng = np.random.default_rng(ctx)
    n, p = 3000, 11
    T = texts.random_text(n, 4, 2, sep_every=0)
    pid = rng.integers(0, p, n).astype(np.uint16)
    retired = (rng.random(n) < 0.3).astype(np.uint8)
    bits = oracle_lib.partition_id_bits(p)
    words = oracle_lib.pack_partition_ids(pid, bits)
    oracle_lib.set_retired(words, bits, np.flatnonzero(retired))
    suf = rng.permutation(n)[:1000].astype(np.uint64)
    lanes = oracle_lib.u64_to_sa40(suf)
    keys = np.zeros((suf.size, key_words), dtype=np.uint64)
    beta = np.zeros(suf.size, dtype=np.uint32)
    rc = emu.csa_stage_slab_u16_dev(T.ctypes.data, n, lanes.ctypes.data, suf.size, key_words, words.ctypes.data, p, ctx,
                                    1 if generation0 else 0, keys.ctypes.data if generation0 else None, beta.ctypes.data, None)
    assert rc == 0, emu.csa_last_error()
    want_keys, want_beta = oracle_lib.stage_slab(T, suf, key_words, pid, retired, ctx, generation0)
    assert np.array_equal(beta, want_beta)
    if generation0:
        assert np.array_equal(keys, want_keys)
    # and the way back: the same lanes scattered to a random rank order
    rank = rng.permutation(suf.size).astype(np.uint32)
    out = np.zeros(5 * suf.size, dtype=np.uint8)
    for capacity in (16, suf.size):  # a small handle scatters directly, one that holds the partition buckets it by windows
        out[:] = 0
        h = C.c_void_p()
        assert emu.csa_create(capacity, 1, C.byref(h)) == 0
        rc = emu.csa_scatter_to_rank_order_dev(h, lanes.ctypes.data, rank.ctypes.data, suf.size, out.ctypes.data, None)
        emu.csa_destroy(h)
        assert rc == 0 and np.array_equal(out, oracle_lib.scatter_to_rank_order(lanes, rank)[1]), capacity


class HostArray:
    """In the emulation "device" memory is host memory: the arrays stand for themselves."""

    def __init__(self, a):
        self.a = a
        self.ptr = a.ctypes.data


@pytest.mark.parametrize("packed,ctx,n,p", [(False, 4, 3000, 5), (True, 8, 3000, 300), (True, 64, 1500, 2049)])
def test_emulated_message_kernels_match_the_oracle(emu, packed, ctx, n, p):
    import test_gpu_messages
    test_gpu_messages.check_messages(emu, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a.copy(), n, p, ctx, packed,
                                     seed=n + p)


def test_emulated_join_matches_the_oracle(emu):
    rng = np.random.default_rng(4)
    n = 2000
    suf = np.sort(rng.choice(1 << 20, n, replace=False)).astype(np.uint64)
    sa = suf | (rng.integers(0, 1 << 16, n).astype(np.uint64) << np.uint64(48))
    primary = rng.integers(0, 1 << 31, n).astype(np.uint32)
    tgt = np.concatenate([suf[rng.choice(n, 700, replace=False)], np.setdiff1d(rng.integers(0, 1 << 20, 200).astype(np.uint64), suf)])
    rank = rng.integers(0, 1 << 32, tgt.size, dtype=np.uint64).astype(np.uint32)
    seed_keys = np.full(n, np.uint64(0xFFFFFFFFFFFFFFFF))
    keys = seed_keys.copy()
    lanes = oracle_lib.u64_to_sa40(tgt)
    assert emu.csa_join_messages_dev(lanes.ctypes.data, rank.ctypes.data, tgt.size, sa.ctypes.data, primary.ctypes.data,
                                     keys.ctypes.data, n, None) == 0
    assert np.array_equal(keys, oracle_lib.join_messages(tgt, rank, sa, primary, seed_keys))
    keys2 = seed_keys.copy()
    h = C.c_void_p()
    assert emu.csa_create(tgt.size, 1, C.byref(h)) == 0
    rc = emu.csa_join_messages_sorted_dev(h, lanes.ctypes.data, rank.ctypes.data, tgt.size, sa.ctypes.data, primary.ctypes.data,
                                          keys2.ctypes.data, n, None)
    emu.csa_destroy(h)
    assert rc == 0 and np.array_equal(keys2, keys)


@pytest.mark.parametrize("p,key_words,sigma,n", [(3, 1, 3, 3000), (7, 2, 2, 2500), (5, 1, 1, 400), (4, 1, 2, 2000)])
def test_multi_partition_pipeline_through_the_emulated_stage_kernels(emu, p, key_words, sigma, n):
    """Partitions that exchange ranks only through messages: every exported stage kernel (partition ids, slab staging,
    message count / offsets / emission, join, rank-order scatter) in the reference's order of use; the suffix array that
    comes out must be the oracle's."""
    import multi_partition
    T = texts.random_text(n, sigma, 11 * p + n, sep_every=0)
    T[-7:] = 0
    if n == 2000:  # long repeats: many generations, pills forwarded over several of them
        T[700:1300] = T[:600]
        T[1500:1900] = T[100:500]
    log = []
    sa, gens = multi_partition.build_sa(emu, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a, T, p, key_words=key_words,
                                        log=log)
    assert np.array_equal(sa, oracle_lib.sa40_to_u64(oracle_lib.build_sa40(T))), (p, key_words, gens)
    assert gens >= 2
    if n == 2000:
        assert gens >= 6 and sum(step[5] for step in log if step[0] >= 1) > 0  # pills travelled in later generations


@pytest.mark.parametrize("p,key_words,sigma,n", [(5, 4, 2, 600), (3, 1, 2, 700)])
def test_multi_partition_pipeline_with_the_emulated_step_entries(emu, p, key_words, sigma, n):
    """The same pipeline with each partition step as one call of csa_sort_init_dev / csa_sort_rerank_dev."""
    import multi_partition
    T = texts.random_text(n, sigma, 13 * p + n, sep_every=0)
    T[-7:] = 0
    if key_words == 1:  # long repeats: many generations, pills forwarded
        T[250:450] = T[:200]
        T[500:650] = T[100:250]
    log, glue_log = [], []
    sa, gens = multi_partition.build_sa(emu, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a, T, p, key_words=key_words,
                                        log=log, step_handle=steps_handle(emu, key_words))
    assert np.array_equal(sa, oracle_lib.sa40_to_u64(oracle_lib.build_sa40(T))), (p, key_words, gens)
    # the same run with numpy glue between the stages: the same cohorts, survivors and message counts at every step
    multi_partition.build_sa(emu, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a, T, p, key_words=key_words, log=glue_log)
    assert log == glue_log


def test_random_pipelines_through_the_emulated_entries(emu):
    """Random texts (tiny alphabets, long repeats, runs of one symbol, zero tails), 1 to 40 partitions, all four key widths,
    through the device-buffer entries and the slab-shaped ones: every step passes the reference's validators inside the
    harness and the suffix array is the oracle's."""
    import multi_partition
    rng = np.random.default_rng(2024)
    for case in range(16):
        n = int(rng.integers(40, 1400))
        sigma = int(rng.choice([1, 2, 3, 5, 40, 65536]))
        T = rng.integers(0, sigma, n).astype(np.uint16)
        shape = case % 4
        if shape == 1 and n > 200:
            length = int(rng.integers(10, n // 2))
            T[n - length:] = T[:length]
        if shape == 2:
            T[-int(rng.integers(1, 30)):] = 0
        if shape == 3 and n > 300:
            a = int(rng.integers(0, n // 2))
            T[a:a + n // 3] = T[a]
        p = int(rng.choice([1, 2, 3, 7, 16, 40]))
        key_words = 1 + case % 4
        kw = {"step_handle": steps_handle(emu, key_words)} if (case // 4) % 2 == 0 else {
            "slab_handle": steps_handle(emu, key_words), "host_buf": lambda nbytes: np.zeros(nbytes, dtype=np.uint8), "chunk_cap": 4096}
        sa, _ = multi_partition.build_sa(emu, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a, T, p, key_words=key_words, seed=case, **kw)
        want, _ = oracle_lib.prefix_doubling(T, 1)
        assert np.array_equal(sa, want), (case, n, sigma, p, key_words)


@pytest.mark.skipif(not os.path.exists(oracle_lib.SA_STRUCTURE), reason="oracle/_ref/sa_structure is not built (make -C oracle, with the reference tree present)")
@pytest.mark.parametrize("p,key_words,pivot_words", [(4, 1, 1), (5, 2, 2), (3, 4, 2)])
def test_the_references_own_predictor_gives_the_cohorts_and_pill_receipts_of_the_steps(emu, tmp_path, p, key_words, pivot_words):
    """The reference's src/sa_structure.cpp predicts a run from the finished suffix array, the key and pivot widths and the
    partition sizes: every generation's active-set size, every query's look-back (how long ago its target retired), and the
    messages emitted before any is withheld from a recipient that is flagged retired. The partition steps of the library
    (one csa_sort_init_dev / csa_sort_rerank_dev call each, on the emulated kernels) must have had exactly those cohorts
    and exactly that many members joined by a pill (csa_step_result.pills, counted on the device), summed over the
    partitions; they emit that many messages in generation 0, when nothing is flagged yet, and never more later."""
    import multi_partition
    T = texts.random_text(800, 2, 17 * p, sep_every=0)
    T[300:520] = T[20:240]
    T[-6:] = 0
    log = []
    sa, _ = multi_partition.build_sa(emu, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a, T, p, key_words=key_words,
                                     pivot_words=pivot_words, seed=p, log=log, step_handle=steps_handle(emu, key_words))
    assert np.array_equal(sa, oracle_lib.sa40_to_u64(oracle_lib.build_sa40(T)))
    ours, theirs = multi_partition.structure_of_a_pipeline_run(T, p, key_words, pivot_words, p, log, multi_partition.build_sa.pill_receipts, tmp_path)
    assert ours["cohorts"] == theirs["cohorts"], (ours, theirs)
    assert ours["pill_receipts"] == theirs["pill_receipts"], (ours, theirs)
    assert ours["messages"][0] == theirs["messages"][0] and all(a <= b for a, b in zip(ours["messages"], theirs["messages"])), (ours, theirs)
    assert len(ours["cohorts"]) >= 4 and sum(ours["pill_receipts"]) > 0


@pytest.mark.parametrize("p,key_words,sigma,n,chunk_cap", [(3, 1, 3, 900, 4096)])
def test_multi_partition_pipeline_through_the_emulated_slab_entries(emu, p, key_words, sigma, n, chunk_cap):
    """csa_sort_init_slabs / csa_sort_rerank_slabs / csa_scatter_slabs: every partition step takes and returns host slabs of
    ragged sizes (several per partition, some empty, the inbox shared out over them), the final permutation comes back cut
    into disk blocks and edges; the suffix array assembled from those pieces is the oracle's."""
    import multi_partition
    T = texts.random_text(n, sigma, 31 * p + n, sep_every=0)
    T[n // 3:n // 3 + 250] = T[:250]
    T[-5:] = 0
    # slabs far smaller than the reference's: a partition of a few thousand suffixes still spans several
    sa, gens = multi_partition.build_sa(emu, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a, T, p, key_words=key_words,
                                        slab_handle=steps_handle(emu, key_words), host_buf=lambda nbytes: np.zeros(nbytes, dtype=np.uint8),
                                        chunk_cap=chunk_cap)
    want, _ = oracle_lib.prefix_doubling(T, key_words)
    assert np.array_equal(sa, want) and gens >= 5


@pytest.mark.parametrize("key_words,p,slabs", [(1, 1, True), (2, 1, True), (3, 2, False), (4, 1, True)])
def test_the_steps_stay_inside_the_floor_plan(emu, key_words, p, slabs):
    """A handle made by csa_create_steps for exactly the largest partition holds csa_step_bytes_per_suffix(key_words)
    bytes per suffix and nothing more is ever allocated: every step of a whole build, slab traffic included, must find
    its columns in that block (a step that does not returns an error naming the column). Texts with long ties on the
    first key word, so that the wide-key path sorts nearly every suffix a second time (its busiest moment). The
    reference's own floor plan is 65 / 65 / 81 / 97 bytes per suffix (src/GPU_SACA.cu:372)."""
    import multi_partition
    per_suffix = int(emu.csa_step_bytes_per_suffix(key_words))
    assert per_suffix == {1: 48, 2: 65, 3: 76, 4: 84}[key_words]
    assert per_suffix <= 2 * (max(8 * key_words, 16) + 8 + 4 + 4) + 1  # the reference's own figure
    for n, sigma in ((420, 2),):
        T = texts.random_text(n, sigma, 5 * n + key_words, sep_every=0)
        kw = {"slab_handle": steps_handle(emu, key_words), "host_buf": lambda nbytes: np.zeros(nbytes, dtype=np.uint8),
              "chunk_cap": 4096} if slabs else {"step_handle": steps_handle(emu, key_words)}
        sa, gens = multi_partition.build_sa(emu, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a, T, p, key_words=key_words, **kw)
        want, _ = oracle_lib.prefix_doubling(T, key_words)
        assert np.array_equal(sa, want), (n, sigma, gens)
        if slabs and p == 1:
            # the busiest step held no more than the documented figure (the partition's size is rounded up to 256 suffixes)
            assert multi_partition.build_sa.high_water <= per_suffix * (n + 255), (multi_partition.build_sa.high_water, per_suffix * n)


def test_sizing_by_the_mirrors_bound_never_exceeds_the_device(emu):
    """What include/cascade_gpu_saca.hpp's partition_size_upper_bound computes (restated here): STREAM_C handles of the
    bound's size, workspaces included, fit into the free memory with the reference's margins."""
    STREAM_C, MARGIN, SLACK = 3, 0.1, 1.20
    for key_words in (1, 2, 3, 4):
        per_suffix = int(emu.csa_step_bytes_per_suffix(key_words))
        for free in (1 << 24, 5 << 30, 96 << 30, 288 << 30):
            budget = int(free * (1.0 - MARGIN) / SLACK)
            sz = min(budget // (STREAM_C * per_suffix), _native.CSA_MAX_PART_SZ)
            while sz > 0 and STREAM_C * (sz * per_suffix + int(emu.csa_workspace_bytes(sz))) > budget:
                ws = STREAM_C * int(emu.csa_workspace_bytes(sz))
                nxt = 0 if ws >= budget else (budget - ws) // (STREAM_C * per_suffix)
                sz = nxt if nxt < sz else sz - 1
            assert STREAM_C * (sz * per_suffix + int(emu.csa_workspace_bytes(sz))) <= budget < free
            if free >= 5 << 30:
                assert sz > 0.8 * budget / (STREAM_C * per_suffix)  # the workspace is a small share


def test_step_entries_on_a_text_of_one_symbol(emu):
    """One symbol: a single group that only sheds its last members each generation; every pivot is equal, so all but
    one partition are empty. Closed form: the shorter suffix comes first."""
    import multi_partition
    T = np.full(100, 9, dtype=np.uint16)
    sa, gens = multi_partition.build_sa(emu, lambda a: HostArray(np.array(a, copy=True)), lambda d: d.a, T, 3, step_handle=steps_handle(emu, 1))
    assert np.array_equal(sa, np.arange(T.size - 1, -1, -1, dtype=np.uint64)), gens


def test_chunked_tile_order_without_resident_workgroups_ends_in_an_error_not_a_hang(emu):
    # The XCD-chunked tile order of the radix pass waits for tiles whose workgroups are dispatched later. The emulator
    # runs one workgroup at a time, the extreme case of a device shared with other launches: the wait must run into
    # its spin limit, every later workgroup and kernel of the step must leave at once, and the call must report
    # CSA_ERR_INTERNAL. By default (no csa_set_device_exclusive) tiles are numbered by arrival and the same text sorts.
    emu.csa_set_device_exclusive.argtypes = [C.c_void_p, C.c_int]
    emu.csa_set_tuning.argtypes = [C.c_void_p, C.c_int, C.c_uint32]
    T = texts.random_text(140000, 5, 3, sep_every=0)  # 137 tiles of 1024 keys: one whole group of 8 chunks of 16
    n = T.size
    h = C.c_void_p()
    # the emulated device has one compute unit: the chunked order is neither offered nor accepted as a tuning value
    assert emu.csa_create(16, 1, C.byref(h)) == 0
    assert emu.csa_set_tuning(h, _native.CSA_TUNE_XCD_CHUNK, 16) == _native.CSA_ERR_ARG and b"compute units" in emu.csa_last_error()
    emu.csa_destroy(h)
    # a device that claims 256 compute units while its workgroups still run one at a time
    os.environ["HIPEMU_CU_COUNT"] = "256"
    try:
        assert emu.csa_create(n, 1, C.byref(h)) == 0
    finally:
        del os.environ["HIPEMU_CU_COUNT"]
    out = np.zeros(5 * n + 8, dtype=np.uint8)
    st = _native.CsaStats()
    try:
        assert emu.csa_set_tuning(h, _native.CSA_TUNE_XCD_CHUNK, 16) == 0
        assert emu.csa_set_tuning(h, _native.CSA_TUNE_XCD_CHUNK, 17) == _native.CSA_ERR_ARG  # 2 * 8 * 17 > 256
        assert emu.csa_set_device_exclusive(h, 1) == 0
        rc = emu.csa_sort_partition_u16_dev(h, T.ctypes.data, n, 0, out.ctypes.data, None, 0, C.byref(st))
        assert rc == -4 and b"spin limit" in emu.csa_last_error(), (rc, emu.csa_last_error())
        assert emu.csa_set_device_exclusive(h, 0) == 0
        small = T[:6000].copy()
        rc = emu.csa_sort_partition_u16_dev(h, small.ctypes.data, small.size, 0, out.ctypes.data, None, 0, C.byref(st))
        assert rc == 0, emu.csa_last_error()
        assert np.array_equal(out[:5 * small.size], oracle_lib.build_sa40(small))
    finally:
        emu.csa_destroy(h)
