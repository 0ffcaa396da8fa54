"""Pins the CPU oracle (oracle/cascade_oracle.c) against the reference's known answers, closed forms,
golden vectors produced by the reference's own compiled CPU sort, and independent rules. CPU only."""
import hashlib
import os

import numpy as np
import pytest

import oracle_lib
import texts

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def sa_of(T):
    return oracle_lib.sa40_to_u64(oracle_lib.build_sa40(T))


def naive_sa(T):
    """Independent definition: tuples compare exactly like "numeric symbols, shorter first"."""
    T = [int(x) for x in T]
    return sorted(range(len(T)), key=lambda i: T[i:])


# ---- sa40 layout -------------------------------------------------------------------------------

def test_sa40_bytes_and_round_trip():
    lib = oracle_lib.oracle()
    buf = np.zeros(5 * 4 + 8, dtype=np.uint8)
    vals = [0, 1, 0x0102030405, (1 << 40) - 1]
    for r, v in enumerate(vals):
        lib.orc_sa40_store(buf.ctypes.data, r, v)
    assert list(buf[10:15]) == [5, 4, 3, 2, 1]  # little-endian, 5 bytes, no gaps
    assert list(buf[15:20]) == [255] * 5 and not buf[20:].any()
    assert [lib.orc_sa40_load(buf.ctypes.data, r) for r in range(4)] == vals
    assert list(oracle_lib.sa40_to_u64(buf[:20])) == vals
    assert bytes(oracle_lib.u64_to_sa40(np.array(vals, dtype=np.uint64))) == bytes(buf[:20])


# ---- order convention --------------------------------------------------------------------------

def test_known_answer_numeric_high_bit_order():
    # the reference's known answer uses uint32 symbols {0x80000000, 0x7FFFFFFF, 0xFFFFFFFF, 0} -> [3, 1, 0, 2]
    # (src/test_query.cu:405-411); the same order statistics in uint16
    assert list(sa_of([0x8000, 0x7FFF, 0xFFFF, 0])) == [3, 1, 0, 2]


def test_shorter_suffix_first_and_zero_tail():
    assert list(sa_of([0, 0, 0, 0])) == [3, 2, 1, 0]
    assert list(sa_of([5, 3, 5, 0])) == [3, 1, 2, 0]  # [0] < [3,5,0] < [5,0] < [5,3,5,0]
    assert list(sa_of([9, 8, 7])) == [2, 1, 0]
    assert list(sa_of([65535, 65535])) == [1, 0]
    T = texts.zero_tail_corner(ell=4)
    n = len(T)
    assert list(sa_of(T)[:4]) == [n - 1, n - 2, n - 3, n - 4]  # dataset/make-corner-case.py:37


def test_closed_forms():
    n = 257
    assert list(sa_of([4] * n)) == list(range(n - 1, -1, -1))
    assert list(sa_of(range(n))) == list(range(n))
    assert list(sa_of(range(n, 0, -1))) == list(range(n - 1, -1, -1))
    # (ab)^k, a < b, ends in b: the a-suffixes shortest first, then the b-suffixes shortest first
    k = 50
    T = texts.periodic(2 * k)
    assert list(sa_of(T)) == list(range(2 * k - 2, -1, -2)) + list(range(2 * k - 1, -1, -2))


def test_byte_order_differs_from_numeric_order():
    # 0x0100 < 0x0201 numerically, but its little-endian bytes (00 01) sort before (01 00) = 0x0001
    T = np.array([0x0100, 0x0001, 0x0201], dtype=np.uint16)
    assert list(sa_of(T)) == [1, 0, 2]


@pytest.mark.parametrize("seed", range(6))
def test_against_naive_definition(seed):
    rng = np.random.default_rng(seed)
    for n in (1, 2, 5, 64, 300):
        T = rng.integers(0, [2, 3, 4, 70000][seed % 4], size=n).astype(np.uint16)
        assert list(sa_of(T)) == naive_sa(T)


def test_cmp_suffixes_contract():
    lib = oracle_lib.oracle()
    T = np.array([1, 2, 1, 2, 1], dtype=np.uint16)
    p = T.ctypes.data
    assert lib.orc_cmp_suffixes_u16(p, 5, 0, 2, 5) == 1   # [1,2,1,2,1] vs its prefix [1,2,1]
    assert lib.orc_cmp_suffixes_u16(p, 5, 2, 0, 5) == -1
    assert lib.orc_cmp_suffixes_u16(p, 5, 0, 2, 2) == 0   # undecided within 2 symbols
    assert lib.orc_cmp_suffixes_u16(p, 5, 0, 2, 3) == -1 or lib.orc_cmp_suffixes_u16(p, 5, 0, 2, 3) == 1
    assert lib.orc_cmp_suffixes_u16(p, 5, 1, 0, 5) == 1
    ref = oracle_lib.ref()
    if ref is not None:
        for i in range(5):
            for j in range(5):
                if i != j:
                    for mc in (1, 2, 3, 5):
                        assert lib.orc_cmp_suffixes_u16(p, 5, i, j, mc) == ref.ref_cmp_suffixes_u16(p, 5, i, j, mc)


# ---- golden vectors from the reference's compiled CPU sort -------------------------------------

def test_golden_fixtures_match_oracle():
    g = np.load(os.path.join(GOLDEN, "fixtures.npz"), allow_pickle=False)
    names = sorted(k[:-5] for k in g.files if k.endswith(".text"))
    assert len(names) >= 70
    for name, T in texts.fixture_suite():
        assert np.array_equal(g[f"{name}.text"], T), f"{name}: the seeded input changed"
        assert np.array_equal(oracle_lib.build_sa40(T), g[f"{name}.sa40"]), name


def test_c1_digest():
    from cascade_amd import workloads
    want = dict(line.split() for line in open(os.path.join(GOLDEN, "c1_sha256.txt")))
    T = workloads.generate(1)
    assert hashlib.sha256(T.tobytes()).hexdigest() == want["text"]
    sa, _ = oracle_lib.prefix_doubling(T, 1)
    assert hashlib.sha256(oracle_lib.u64_to_sa40(sa).tobytes()).hexdigest() == want["sa40"]


def test_reference_library_agrees_when_present():
    ref = oracle_lib.ref()
    if ref is None:
        pytest.skip("oracle/_ref was not built here")
    for seed in range(4):
        T = texts.random_text(3000, [2, 4, 256, 65536][seed], 77 + seed)
        assert np.array_equal(oracle_lib.build_sa40(T), oracle_lib.build_sa40(T, lib=ref))
        sa = oracle_lib.sa40_to_u64(oracle_lib.build_sa40(T))
        assert ref.ref_is_correct_sa_u16(sa.ctypes.data, T.ctypes.data, T.size) == 1
        w = np.array([1, 2, 3, 4], dtype=np.uint16)
        assert ref.ref_pack_word_u16(w.ctypes.data) == oracle_lib.oracle().orc_pack_word_u16(w.ctypes.data)
    for n in (1, 3, 4, 5, 100):
        for ell in (4, 8):
            for j in range(n):
                assert ref.ref_fwd_tag_single_partition(j + ell, n, ell) == oracle_lib.oracle().orc_fwd_tag(j + ell, n, ell)


# ---- verifier -----------------------------------------------------------------------------------

def test_verifier_accepts_truth_and_rejects_controls():
    rng = np.random.default_rng(5)
    T = np.where(rng.integers(0, 4, 4000) == 0, 0x0100, np.where(rng.integers(0, 2, 4000) == 1, 0x0001, 0x0201)).astype(np.uint16)
    n = T.size
    sa = sa_of(T)
    assert oracle_lib.is_correct_sa(sa, T)
    assert oracle_lib.is_correct_sa40(oracle_lib.u64_to_sa40(sa), T)
    # byte-order suffix array (the negative control of src/test_query.cu:417-433)
    B = T.view(np.uint8).reshape(n, 2)
    byte_sa = np.array(sorted(range(n), key=lambda i: bytes(B[i:].reshape(-1))), dtype=np.uint64)
    assert not oracle_lib.is_correct_sa(byte_sa, T)
    swapped = sa.copy()
    swapped[[100, 101]] = swapped[[101, 100]]
    assert not oracle_lib.is_correct_sa(swapped, T)
    oob = sa.copy()
    oob[7] = n + 3
    assert not oracle_lib.is_correct_sa(oob, T)
    rep = sa.copy()
    rep[11] = rep[10]
    assert not oracle_lib.is_correct_sa(rep, T)
    assert oracle_lib.is_correct_sa(np.zeros(0, dtype=np.uint64), np.zeros(0, dtype=np.uint16))


# ---- key packing and the tail tag -----------------------------------------------------------------

def test_pack_word_closed_form_and_order_invariant():
    lib = oracle_lib.oracle()
    w = np.array([0x1234, 0xABCD, 0x0001, 0xFFFF], dtype=np.uint16)
    assert lib.orc_pack_word_u16(w.ctypes.data) == 0x1234ABCD0001FFFF
    T = texts.random_text(500, 4, 3)
    for kw in (1, 2):
        K = oracle_lib.pack_prefix(T, kw)
        assert np.array_equal(K, oracle_lib.pack_prefix_np(T, kw))
        P = np.concatenate([T, np.zeros(4 * kw, dtype=np.uint16)])
        rng = np.random.default_rng(1)
        for _ in range(2000):
            i, j = rng.integers(0, T.size, 2)
            ki, kj = tuple(K[i]), tuple(K[j])
            ti, tj = tuple(P[i:i + 4 * kw]), tuple(P[j:j + 4 * kw])
            assert (ki < kj) == (ti < tj) and (ki == kj) == (ti == tj)
    # tail: positions past the end read as zero
    K = oracle_lib.pack_prefix(np.array([7, 8], dtype=np.uint16), 1)
    assert [int(k) for k in K[:, 0]] == [0x0007000800000000, 0x0008000000000000]


def test_fwd_tag_closed_form():
    lib = oracle_lib.oracle()
    n, ell = 100, 4
    tags = [lib.orc_fwd_tag(j + ell, n, ell) for j in range(n)]
    assert tags[:n - ell] == [ell] * (n - ell)
    assert tags[n - ell:] == [3, 2, 1, 0]  # the shorter the suffix, the smaller its tag


# ---- prefix doubling restatement ------------------------------------------------------------------

@pytest.mark.parametrize("key_words", [1, 2])
def test_prefix_doubling_equals_comparison_sort(key_words):
    for name, T in texts.fixture_suite():
        sa, counts = oracle_lib.prefix_doubling(T, key_words)
        assert np.array_equal(sa, sa_of(T)), name
        assert counts[0] == len(T)


@pytest.mark.parametrize("key_words", [1, 2])
def test_active_counts_follow_the_retirement_rule(key_words):
    # independent closed form over the finished SA and LCPs (src/sa_structure.cpp:295-306,375)
    ell = 4 * key_words
    cases = [texts.random_text(3000, 2, 1, sep_every=0), texts.random_text(3000, 4, 2), texts.periodic(600),
             texts.fibonacci_word(800), texts.zero_tail_corner(2000), np.zeros(300, dtype=np.uint16)]
    for T in cases:
        sa, counts = oracle_lib.prefix_doubling(T, key_words)
        d = oracle_lib.retire_generations(T, sa, ell)
        want = [len(T)] + [int((d >= g).sum()) for g in range(1, int(d.max()) + 1)]
        assert counts == want


def test_stable_sort_pairs_contract():
    rng = np.random.default_rng(0)
    keys = rng.integers(0, 1 << 20, 5000).astype(np.uint64) << np.uint64(7)
    vals = np.arange(5000, dtype=np.uint32)
    k, v = oracle_lib.stable_sort_pairs(keys, vals, 7, 27)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(k, keys[order]) and np.array_equal(v, vals[order])
    k, v = oracle_lib.stable_sort_pairs(keys, vals, 7, 15)  # a sub-range of the bits only
    order = np.argsort((keys >> np.uint64(7)) & np.uint64(0xFF), kind="stable")
    assert np.array_equal(k, keys[order]) and np.array_equal(v, vals[order])


SA_CONVERT = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref", "sa_convert")


@pytest.mark.skipif(not os.path.exists(SA_CONVERT), reason="oracle/_ref/sa_convert is not built (make -C oracle, with the reference tree present)")
def test_the_references_own_tool_accepts_and_widens_the_oracles_suffix_array_file(tmp_path):
    """The reference's tools/sa_convert.cpp, compiled from its one source file (oracle/Makefile): `--meta-only` is what the
    reference runs on a finished 40-bit suffix array (file of 5 n bytes beside a text of n symbols, a spot check of the
    order of adjacent entries with its own comparator, index.meta), `--widen` reads the 5-byte entries with its own
    sa40 loader. The oracle's file must pass the first and widen to the oracle's 64-bit array; a file with two entries
    swapped, and one that is an entry short, must be refused. Pins the on-disk layout of the output row."""
    import subprocess
    for name, T in (("tokens", texts.random_text(30000, 50257, 3, sep_every=700)), ("ties", texts.random_text(5000, 2, 4, sep_every=0))):
        text, sa = tmp_path / f"{name}.u16", tmp_path / f"{name}.u40"
        T.astype("<u2").tofile(text)
        sa40 = oracle_lib.build_sa40(T)
        sa40.tofile(sa)
        idx = tmp_path / f"{name}.index"
        r = subprocess.run([SA_CONVERT, "--meta-only", "--sa", str(sa), "--text", str(text), "--sym-bytes", "2", "--index-dir", str(idx)],
                           capture_output=True, text=True, timeout=120)
        assert r.returncode == 0 and "spot-check passed" in r.stderr, r.stderr
        assert (idx / "index.meta").exists()
        wide = tmp_path / f"{name}.u64"
        r = subprocess.run([SA_CONVERT, "--widen", "--in", str(sa), "--out", str(wide)], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stderr
        assert np.array_equal(np.fromfile(wide, dtype="<u8"), oracle_lib.sa40_to_u64(sa40))
        bad = sa40.copy()
        bad[5 * 100:5 * 101], bad[5 * 101:5 * 102] = sa40[5 * 101:5 * 102].copy(), sa40[5 * 100:5 * 101].copy()
        bad.tofile(sa)
        r = subprocess.run([SA_CONVERT, "--meta-only", "--sa", str(sa), "--text", str(text), "--sym-bytes", "2", "--index-dir", str(idx)],
                           capture_output=True, text=True, timeout=120)
        assert r.returncode != 0, "two swapped entries passed the order check"
        sa40[:-5].tofile(sa)
        r = subprocess.run([SA_CONVERT, "--meta-only", "--sa", str(sa), "--text", str(text), "--sym-bytes", "2", "--index-dir", str(idx)],
                           capture_output=True, text=True, timeout=120)
        assert r.returncode != 0, "a file one entry short passed"


@pytest.mark.skipif(not os.path.exists(oracle_lib.SA_STRUCTURE), reason="oracle/_ref/sa_structure is not built (make -C oracle, with the reference tree present)")
@pytest.mark.parametrize("key_words", [1, 2, 3, 4])
def test_generation_sizes_are_those_the_references_own_predictor_gives(tmp_path, key_words):
    """The reference's src/sa_structure.cpp, compiled from its one source file (oracle/Makefile), predicts from a finished
    suffix array how many suffixes retire at every generation of a run (and checks the array on the way). The oracle's
    prefix doubling must report exactly those active-set sizes, for every key width, on texts with deep repeats, runs and
    a tail of zeros. Pins orc_prefix_doubling's per-generation counts on the reference's code instead of on the
    restatement of its rule (orc_retire_generations)."""
    ell = 4 * key_words
    rng = np.random.default_rng(key_words)
    cases = {"tokens": texts.random_text(20000, 50257, 3, sep_every=500), "ties": texts.random_text(20000, 3, 5, sep_every=0),
             "run": np.concatenate([texts.random_text(3000, 4, 6, sep_every=0), np.full(5000, 2, dtype=np.uint16),
                                    texts.random_text(3000, 4, 7, sep_every=0)]).astype(np.uint16)}
    cases["tokens"][12000:18000] = cases["tokens"][1000:7000]
    cases["ties"][15000:19000] = cases["ties"][2000:6000]
    cases["ties"][-9:] = 0
    for name, T in cases.items():
        sa, counts = oracle_lib.prefix_doubling(T, key_words)
        got = oracle_lib.reference_structure(T, oracle_lib.u64_to_sa40(sa), ell, ell, [T.size], tmp_path)
        assert got["n"] == T.size and got["ell"] == ell
        assert oracle_lib.active_sizes_from_retirements(T.size, got["retire_hist"]) == counts, name
