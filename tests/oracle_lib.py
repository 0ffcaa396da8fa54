"""ctypes access to the CPU oracle (oracle/_build/libcascade_oracle.so) and, where it was built, to the
reference's own CPU oracle (oracle/_ref/libcascade_ref.so). Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "_build", "libcascade_oracle.so")
REF_LIB = os.path.join(ORACLE_DIR, "_ref", "libcascade_ref.so")
SA_PAD = 128

_oracle = None
_ref = None


def oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_LIB):
            subprocess.run(["make", "-C", ORACLE_DIR, "_build/libcascade_oracle.so"], check=True)
        lib = C.CDLL(ORACLE_LIB)
        vp, u64, i32 = C.c_void_p, C.c_uint64, C.c_int
        lib.orc_cmp_suffixes_u16.restype = i32
        lib.orc_cmp_suffixes_u16.argtypes = [vp, u64, u64, u64, u64]
        lib.orc_sa40_store.restype = None
        lib.orc_sa40_store.argtypes = [vp, u64, u64]
        lib.orc_sa40_load.restype = u64
        lib.orc_sa40_load.argtypes = [vp, u64]
        lib.orc_build_sa40_u16.restype = None
        lib.orc_build_sa40_u16.argtypes = [vp, u64, vp]
        lib.orc_is_permutation.restype = i32
        lib.orc_is_permutation.argtypes = [vp, u64]
        lib.orc_is_correct_sa_u16.restype = i32
        lib.orc_is_correct_sa_u16.argtypes = [vp, vp, u64]
        lib.orc_is_correct_sa40_u16.restype = i32
        lib.orc_is_correct_sa40_u16.argtypes = [vp, vp, u64]
        lib.orc_pack_word_u16.restype = u64
        lib.orc_pack_word_u16.argtypes = [vp]
        lib.orc_pack_prefix_u16.restype = None
        lib.orc_pack_prefix_u16.argtypes = [vp, u64, u64, i32, vp]
        lib.orc_fwd_tag.restype = u64
        lib.orc_fwd_tag.argtypes = [u64, u64, u64]
        lib.orc_prefix_doubling_u16.restype = i32
        lib.orc_prefix_doubling_u16.argtypes = [vp, u64, i32, vp, vp, i32]
        lib.orc_retire_generations_u16.restype = None
        lib.orc_retire_generations_u16.argtypes = [vp, u64, vp, u64, vp]
        lib.orc_stable_sort_pairs_u64_u32.restype = None
        lib.orc_stable_sort_pairs_u64_u32.argtypes = [vp, vp, u64, i32, i32]
        u32 = C.c_uint32
        lib.orc_partition_id_bits.restype = u32
        lib.orc_partition_id_bits.argtypes = [u32]
        lib.orc_partition_ids_u16.restype = None
        lib.orc_partition_ids_u16.argtypes = [vp, u64, u64, vp, i32, u32, vp, vp]
        lib.orc_pack_partition_ids.restype = None
        lib.orc_pack_partition_ids.argtypes = [vp, u64, u32, vp]
        lib.orc_partition_id_map_get.restype = C.c_uint16
        lib.orc_partition_id_map_get.argtypes = [vp, u32, u64]
        lib.orc_stage_slab_u16.restype = None
        lib.orc_stage_slab_u16.argtypes = [vp, u64, vp, u64, i32, vp, vp, u64, i32, vp, vp]
        lib.orc_messages_of.restype = None
        lib.orc_messages_of.argtypes = [u64, u64, u32, u64, u64, u64, i32, vp]
        lib.orc_count_messages.restype = None
        lib.orc_count_messages.argtypes = [vp, vp, vp, u64, u64, i32, vp]
        lib.orc_emit_messages.restype = None
        lib.orc_emit_messages.argtypes = [vp, vp, vp, u64, u64, i32, u64, vp, vp, vp]
        lib.orc_join_messages.restype = None
        lib.orc_join_messages.argtypes = [vp, vp, u32, vp, vp, vp, u64]
        lib.orc_scatter_to_rank_order.restype = i32
        lib.orc_scatter_to_rank_order.argtypes = [vp, vp, u64, vp]
        lib.orc_output_cut.restype = None
        lib.orc_output_cut.argtypes = [u64, u64, u64, u64, u64, vp]
        _oracle = lib
    return _oracle


def ref():
    """The reference's own CPU oracle, or None where it was not built (no /root/reference and no prebuilt copy)."""
    global _ref
    if _ref is None and os.path.exists(REF_LIB):
        lib = C.CDLL(REF_LIB)
        vp, u64, i32 = C.c_void_p, C.c_uint64, C.c_int
        lib.ref_build_sa40_u16.restype = None
        lib.ref_build_sa40_u16.argtypes = [vp, u64, vp]
        lib.ref_is_correct_sa_u16.restype = i32
        lib.ref_is_correct_sa_u16.argtypes = [vp, vp, u64]
        lib.ref_cmp_suffixes_u16.restype = i32
        lib.ref_cmp_suffixes_u16.argtypes = [vp, u64, u64, u64, u64]
        lib.ref_pack_word_u16.restype = u64
        lib.ref_pack_word_u16.argtypes = [vp]
        lib.ref_fwd_tag_single_partition.restype = u64
        lib.ref_fwd_tag_single_partition.argtypes = [u64, u64, u64]
        u32 = C.c_uint32
        lib.ref_pivot_words.restype = i32
        lib.ref_pivot_words.argtypes = []
        lib.ref_pivot_key_le_u16.restype = i32
        lib.ref_pivot_key_le_u16.argtypes = [vp, vp]
        lib.ref_partition_id_bits.restype = u32
        lib.ref_partition_id_bits.argtypes = [u32]
        lib.ref_partition_id_pack.restype = None
        lib.ref_partition_id_pack.argtypes = [vp, u64, u32, vp]
        lib.ref_messages_of.restype = None
        lib.ref_messages_of.argtypes = [u64, u64, u32, u64, u64, u64, i32, vp]
        lib.ref_joined_key.restype = u64
        lib.ref_joined_key.argtypes = [u32, u32]
        lib.ref_beta_u16.restype = u32
        lib.ref_beta_u16.argtypes = [u64, u64, u64, u64, i32, vp, vp]
        _ref = lib
    return _ref


def _text(T):
    return np.ascontiguousarray(T, dtype=np.uint16)


def _ptr(a):
    return a.ctypes.data if a.size else None


def build_sa40(T, lib=None):
    """sa40 bytes (5*n, pad stripped) of the text by the oracle's comparison sort (or by `lib` = ref())."""
    T = _text(T)
    n = T.size
    out = np.zeros(5 * n + SA_PAD, dtype=np.uint8)
    if lib is None:
        oracle().orc_build_sa40_u16(_ptr(T), n, out.ctypes.data)
    else:
        lib.ref_build_sa40_u16(_ptr(T), n, out.ctypes.data)
    assert not out[5 * n:].any()
    return out[:5 * n].copy()


def sa40_to_u64(sa40):
    sa40 = np.ascontiguousarray(sa40, dtype=np.uint8)
    n = sa40.size // 5
    b = sa40[:5 * n].reshape(n, 5).astype(np.uint64)
    return b[:, 0] | (b[:, 1] << np.uint64(8)) | (b[:, 2] << np.uint64(16)) | (b[:, 3] << np.uint64(24)) | (
        b[:, 4] << np.uint64(32))


def u64_to_sa40(sa):
    sa = np.ascontiguousarray(sa, dtype=np.uint64)
    out = np.empty((sa.size, 5), dtype=np.uint8)
    for b in range(5):
        out[:, b] = (sa >> np.uint64(8 * b)) & np.uint64(0xFF)
    return out.reshape(-1)


def is_correct_sa(sa, T):
    T = _text(T)
    sa = np.ascontiguousarray(sa, dtype=np.uint64)
    return bool(oracle().orc_is_correct_sa_u16(_ptr(sa), _ptr(T), T.size))


def is_correct_sa40(sa40, T):
    T = _text(T)
    sa40 = np.ascontiguousarray(sa40, dtype=np.uint8)
    assert sa40.size == 5 * T.size
    return bool(oracle().orc_is_correct_sa40_u16(_ptr(sa40), _ptr(T), T.size))


def prefix_doubling(T, key_words=1, max_gens=64):
    T = _text(T)
    n = T.size
    sa = np.zeros(n, dtype=np.uint64)
    counts = np.zeros(max_gens, dtype=np.uint64)
    g = oracle().orc_prefix_doubling_u16(_ptr(T), n, key_words, _ptr(sa), counts.ctypes.data, max_gens)
    return sa, [int(c) for c in counts[:g]]


def retire_generations(T, sa, ell):
    T = _text(T)
    sa = np.ascontiguousarray(sa, dtype=np.uint64)
    d = np.zeros(T.size, dtype=np.uint8)
    oracle().orc_retire_generations_u16(_ptr(T), T.size, _ptr(sa), ell, _ptr(d))
    return d


def pack_prefix(T, key_words=1):
    T = _text(T)
    n = T.size
    out = np.zeros((n, key_words), dtype=np.uint64)
    tmp = np.zeros(key_words, dtype=np.uint64)
    lib = oracle()
    for j in range(n):
        lib.orc_pack_prefix_u16(_ptr(T), n, j, key_words, tmp.ctypes.data)
        out[j] = tmp
    return out


def pack_prefix_np(T, key_words=1):
    """Vectorised form of pack_prefix for large inputs (checked against it in the oracle tests)."""
    T = _text(T)
    n = T.size
    P = np.concatenate([T, np.zeros(4 * key_words, dtype=np.uint16)]).astype(np.uint64)
    out = np.zeros((n, key_words), dtype=np.uint64)
    for w in range(key_words):
        for k in range(4):
            out[:, w] = (out[:, w] << np.uint64(16)) | P[4 * w + k: 4 * w + k + n]
    return out


def stable_sort_pairs(keys, vals, begin_bit=0, end_bit=64):
    keys = np.array(keys, dtype=np.uint64, copy=True)
    vals = np.array(vals, dtype=np.uint32, copy=True)
    oracle().orc_stable_sort_pairs_u64_u32(_ptr(keys), _ptr(vals), keys.size, begin_bit, end_bit)
    return keys, vals


def partition_id_bits(p):
    return int(oracle().orc_partition_id_bits(int(p)))


def partition_ids(T, pivots, p, words, text_len=None, n=None):
    """(pid uint16[n], psz uint64[p]) of the suffixes [0, n) of T (default: all); pivots is a (p - 1, words) uint64 array."""
    T = _text(T)
    n = T.size if n is None else int(n)
    text_len = T.size if text_len is None else int(text_len)
    pivots = np.ascontiguousarray(pivots, dtype=np.uint64).reshape(-1)
    assert pivots.size == (p - 1) * words
    pid = np.zeros(max(n, 1), dtype=np.uint16)
    psz = np.zeros(p, dtype=np.uint64)
    oracle().orc_partition_ids_u16(_ptr(T), n, text_len, _ptr(pivots) if pivots.size else None, int(words), int(p), _ptr(pid),
                                   _ptr(psz))
    return pid[:n], psz


def packed_words(n, bits):
    """Words the packed map of n suffixes occupies up to and including a trailing partial group."""
    return (n // 64) * bits + ((n % 64) * bits + 63) // 64


def pack_partition_ids(pid, bits, fill=0):
    pid = np.ascontiguousarray(pid, dtype=np.uint16)
    out = np.full(((pid.size + 63) // 64) * bits + 1, fill, dtype=np.uint64)
    oracle().orc_pack_partition_ids(_ptr(pid), pid.size, int(bits), _ptr(out))
    return out


def sample_pivots(T, p, words, rng, duplicates=False):
    """p - 1 ascending pivots drawn from the K-grams of T (what the reference's sampler hands over, include/GPU_SACA.hpp:76)."""
    T = _text(T)
    if p <= 1:
        return np.zeros((0, words), dtype=np.uint64)
    pos = rng.integers(0, T.size, p - 1)
    if duplicates and p > 3:
        pos[1::3] = pos[0:-1:3][:pos[1::3].size]
    keys = pack_prefix_np(T, words).reshape(T.size, words)[pos]
    order = np.lexsort(tuple(keys[:, w] for w in reversed(range(words))))
    return np.ascontiguousarray(keys[order])


def scatter_to_rank_order(suf40, rank):
    suf40 = np.ascontiguousarray(suf40, dtype=np.uint8)
    rank = np.ascontiguousarray(rank, dtype=np.uint32)
    out = np.zeros(5 * rank.size, dtype=np.uint8)
    rc = oracle().orc_scatter_to_rank_order(_ptr(suf40), _ptr(rank), rank.size, _ptr(out))
    return rc, out


def output_cut(lo, hi, chunk_bytes, c, chunk_c):
    out = np.zeros(6, dtype=np.uint64)
    oracle().orc_output_cut(int(lo), int(hi), int(chunk_bytes), int(c), int(chunk_c), _ptr(out))
    return [int(v) for v in out]


def stage_slab(T, suf, key_words, pid, retired, ctx, generation0):
    """(keys uint64[count, key_words] or None, beta uint32[count]) for the suffixes `suf` (uint64 array)."""
    T = _text(T)
    suf = np.ascontiguousarray(suf, dtype=np.uint64)
    lanes = u64_to_sa40(suf)
    pid = np.ascontiguousarray(pid, dtype=np.uint16)
    retired = np.ascontiguousarray(retired, dtype=np.uint8)
    keys = np.zeros((suf.size, key_words), dtype=np.uint64) if generation0 else None
    beta = np.zeros(suf.size, dtype=np.uint32)
    oracle().orc_stage_slab_u16(_ptr(T), T.size, _ptr(lanes), suf.size, int(key_words), _ptr(pid), _ptr(retired), int(ctx),
                                1 if generation0 else 0, _ptr(keys) if generation0 else None, _ptr(beta))
    return keys, beta


def set_retired(words, bits, positions):
    """Marks text positions retired in a packed map: the top bit of their entries (include/Partition_ID_Map.hpp:55,198-202)."""
    bit = np.asarray(positions, dtype=np.uint64) * np.uint64(bits) + np.uint64(bits - 1)
    np.bitwise_or.at(words, (bit // np.uint64(64)).astype(np.int64), np.uint64(1) << (bit % np.uint64(64)))


def retired(words, bits, positions):
    """The retirement flags of text positions in a packed map (Partition_ID_Map::retired, include/Partition_ID_Map.hpp:180)."""
    bit = np.asarray(positions, dtype=np.uint64) * np.uint64(bits) + np.uint64(bits - 1)
    return ((words[(bit // np.uint64(64)).astype(np.int64)] >> (bit % np.uint64(64))) & np.uint64(1)).astype(bool)


def count_messages(sa, keys, beta, ctx, packed, p):
    sa, keys = np.ascontiguousarray(sa, dtype=np.uint64), np.ascontiguousarray(keys, dtype=np.uint64)
    beta = np.ascontiguousarray(beta, dtype=np.uint32)
    cnt = np.zeros(p + 1, dtype=np.uint32)
    oracle().orc_count_messages(_ptr(sa), _ptr(keys), _ptr(beta), sa.size, int(ctx), 1 if packed else 0, _ptr(cnt))
    return cnt


def emit_messages(sa, keys, beta, ctx, packed, active_sz, p):
    """(target uint64[total], rank uint32[total], end offsets uint32[p + 1]) with the groups in list order."""
    sa, keys = np.ascontiguousarray(sa, dtype=np.uint64), np.ascontiguousarray(keys, dtype=np.uint64)
    beta = np.ascontiguousarray(beta, dtype=np.uint32)
    cnt = count_messages(sa, keys, beta, ctx, packed, p)
    off = np.zeros(p + 1, dtype=np.uint32)
    off[1:] = np.cumsum(cnt[:-1])
    total = int(cnt.sum())
    tgt = np.zeros(5 * max(total, 1), dtype=np.uint8)
    rank = np.zeros(max(total, 1), dtype=np.uint32)
    oracle().orc_emit_messages(_ptr(sa), _ptr(keys), _ptr(beta), sa.size, int(ctx), 1 if packed else 0, int(active_sz), _ptr(tgt),
                               _ptr(rank), _ptr(off))
    return sa40_to_u64(tgt)[:total], rank[:total], off


def join_messages(msg_target, msg_rank, sa, primary, keys):
    lanes = u64_to_sa40(np.ascontiguousarray(msg_target, dtype=np.uint64))
    msg_rank = np.ascontiguousarray(msg_rank, dtype=np.uint32)
    sa = np.ascontiguousarray(sa, dtype=np.uint64)
    primary = np.ascontiguousarray(primary, dtype=np.uint32)
    keys = np.array(keys, dtype=np.uint64, copy=True)
    oracle().orc_join_messages(_ptr(lanes), _ptr(msg_rank), msg_rank.size, _ptr(sa), _ptr(primary), _ptr(keys), sa.size)
    return keys


SA_STRUCTURE = os.path.join(ORACLE_DIR, "_ref", "sa_structure")


def reference_structure(T, sa40, ell, K, partition_sizes, workdir):
    """What the reference's own src/sa_structure.cpp (compiled from its source into oracle/_ref/sa_structure) predicts for a
    run over the text T with the finished suffix array sa40 (5-byte entries), generation-0 keys of ell symbols, pivots of K
    symbols (0 < K <= ell) and the given partition sizes: a dict with retire_hist[d] (suffixes that retire at generation d),
    payloads[t] and forwards[t] (messages and forwarded pills emitted at generation t) and the rest of its JSON. The tool
    also checks that the array is a permutation in suffix order. None if the tool is not built."""
    import json
    if not os.path.exists(SA_STRUCTURE):
        return None
    workdir = str(workdir)
    text, sa, log, out = (os.path.join(workdir, f) for f in ("structure_text.u16", "structure_sa.u40", "structure_run.log", "structure.json"))
    _text(T).astype("<u2").tofile(text)
    np.ascontiguousarray(sa40, dtype=np.uint8)[:5 * _text(T).size].tofile(sa)
    with open(log, "w") as f:  # the two lines of a STATS build that the tool reads (src/sa_structure.cpp:78-112)
        f.write(f"Pivots selection: {len(partition_sizes)} partitions from 0 samples of {int(K)}-symbol prefixes; initial sort-keys of {int(ell)} symbols.\n")
        f.write("Partition sizes: " + " ".join(str(int(x)) for x in partition_sizes) + "\n")
    run = subprocess.run([SA_STRUCTURE, text, sa, log, out], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    with open(out) as f:
        return json.load(f)


def active_sizes_from_retirements(n, retire_hist):
    """Active-set size entering every generation 0, 1, ... from the retirements per generation, trailing empty ones cut."""
    sizes, left = [], int(n)
    for r in retire_hist:
        sizes.append(left)
        left -= int(r)
    assert left == 0
    while sizes and sizes[-1] == 0:
        sizes.pop()
    return sizes
