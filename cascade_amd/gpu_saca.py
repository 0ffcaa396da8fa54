"""Host-side mirror of the reference's builder interface for the one path this package implements.

Reference: `gpu_saca::GPU_SACA<uint16_t>(ip_path, op_path).build_SA()` (include/GPU_SACA.hpp:304-313,
src/main.cu:12-46) reads a file of little-endian uint16 symbols and writes one 5-byte little-endian suffix
index per symbol, in suffix order. Here the whole text is one partition, sorted in HBM through the C ABI
(include/cascade_hip.h). Where the reference prints a message and exits on an error, these raise.
"""
import ctypes as C

import numpy as np

from . import _native

SA_WIDTH = 5  # include/sa40.hpp:24


def stats_to_dict(st):
    g = int(st.generations)
    return {
        "n": int(st.n),
        "key_words": int(st.key_words),
        "generations": g,
        "active": [int(st.active[i]) for i in range(g)],
        "groups": [int(st.groups[i]) for i in range(g)],
        "big": [int(st.big[i]) for i in range(g)],
        "presorted": [int(st.presorted[i]) for i in range(g)],
        "passes": [int(st.passes[i]) for i in range(g)],
        "rank_update": [int(st.rank_update[i]) for i in range(g)],
        "small_only": [int(st.small_only[i]) for i in range(g)],
        "dense": [int(st.dense[i]) for i in range(g)],
        "ms": [float(st.ms[i]) for i in range(g)],
        "ms_output": float(st.ms_output),
        "ms_total": float(st.ms_total),
        "radix_launches": int(st.radix_launches),
        "radix_pairs": int(st.radix_pairs),
        "radix_ms": float(st.radix_ms),
        "key_symbols": int(st.key_symbols),
        "first_sort_generations": int(st.first_sort_generations),
    }


class PartitionSorter:
    """Owns the device scratch for partitions of up to `max_part_sz` suffixes (csa_create / csa_destroy).
    for_steps: the handle is made by csa_create_steps instead: sized for the per-generation steps
    (csa_step_bytes_per_suffix), without the arrays of the resident sort, which then refuses it."""

    def __init__(self, max_part_sz, key_words=1, device_exclusive=False, for_steps=False):
        self._lib = _native.load()
        self._h = C.c_void_p()
        create = self._lib.csa_create_steps if for_steps else self._lib.csa_create
        _native.check(create(int(max_part_sz), int(key_words), C.byref(self._h)))
        self.max_part_sz = int(max_part_sz)
        self.key_words = int(key_words)
        self.last_stats = None
        if device_exclusive:
            self.set_device_exclusive(True)

    def set_device_exclusive(self, exclusive):
        """Declares that nothing else runs on the device during this handle's calls (csa_set_device_exclusive): the
        radix passes may then use the XCD-chunked tile order, which is not safe next to other launches."""
        _native.check(self._lib.csa_set_device_exclusive(self._h, 1 if exclusive else 0))

    def set_tuning(self, knob, value):
        """One of the thresholds that choose between equivalent ways of doing a step (csa_set_tuning; knob = one of
        _native.CSA_TUNE_*)."""
        _native.check(self._lib.csa_set_tuning(self._h, int(knob), int(value)))

    def close(self):
        if self._h:
            self._lib.csa_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @staticmethod
    def bytes_per_suffix(key_words=1):
        return int(_native.load().csa_bytes_per_suffix(int(key_words)))

    @staticmethod
    def step_bytes_per_suffix(key_words=1):
        return int(_native.load().csa_step_bytes_per_suffix(int(key_words)))

    def scratch_high_water(self):
        """Bytes of the handle's block that the last call held at its busiest moment (csa_scratch_high_water)."""
        return int(self._lib.csa_scratch_high_water(self._h))

    def sort_ptr(self, d_text, n, d_sa40, index_base=0, stream=0, flags=0):
        """Raw device pointers in, statistics out (csa_sort_partition_u16_dev)."""
        st = _native.CsaStats()
        _native.check(self._lib.csa_sort_partition_u16_dev(self._h, d_text, int(n), int(index_base), d_sa40,
                                                           stream or None, int(flags), C.byref(st)))
        self.last_stats = stats_to_dict(st)
        return self.last_stats

    def sort(self, text, out=None, index_base=0, flags=0):
        """text: a uint16 torch tensor on the GPU (viewed as int16 is fine). Returns a uint8 tensor of 5*n bytes."""
        import torch
        assert text.is_cuda and text.element_size() == 2 and text.is_contiguous()
        n = text.numel()
        if out is None:
            out = torch.empty(SA_WIDTH * n + 128, dtype=torch.uint8, device=text.device)  # pad: include/sa40.hpp:31-37
        assert out.is_cuda and out.dtype == torch.uint8 and out.numel() >= SA_WIDTH * n
        stream = torch.cuda.current_stream(text.device).cuda_stream
        self.sort_ptr(text.data_ptr(), n, out.data_ptr(), index_base, stream, flags)
        return out[:SA_WIDTH * n]

    def radix_sort_pairs(self, keys, vals, begin_bit=0, end_bit=64):
        """In-place stable LSD sort of (uint64 key, uint32 value) device tensors (csa_radix_sort_pairs_dev)."""
        import torch
        assert keys.is_cuda and vals.is_cuda and keys.element_size() == 8 and vals.element_size() == 4
        assert keys.numel() == vals.numel()
        stream = torch.cuda.current_stream(keys.device).cuda_stream
        _native.check(self._lib.csa_radix_sort_pairs_dev(self._h, keys.data_ptr(), vals.data_ptr(), keys.numel(),
                                                         int(begin_bit), int(end_bit), stream or None))

    def scatter_to_rank_order(self, suf40, rank, out=None):
        """out lane[rank[i]] = lane i of suf40 (csa_scatter_to_rank_order_dev): uint8 tensor of 5 * m bytes, int32/uint32
        tensor of m ranks (a permutation of [0, m)). Returns the uint8 tensor of 5 * m bytes in rank order."""
        import torch
        m = rank.numel()
        assert suf40.is_cuda and rank.is_cuda and suf40.dtype == torch.uint8 and rank.element_size() == 4
        assert suf40.numel() >= SA_WIDTH * m
        if out is None:
            out = torch.empty(SA_WIDTH * m + 128, dtype=torch.uint8, device=rank.device)
        stream = torch.cuda.current_stream(rank.device).cuda_stream
        _native.check(self._lib.csa_scatter_to_rank_order_dev(self._h, suf40.data_ptr(), rank.data_ptr(), m, out.data_ptr(),
                                                              stream or None))
        return out[:SA_WIDTH * m]

    def verify(self, text, sa40, index_base=0):
        """Device-side O(n) suffix-array check (csa_verify_sa40_dev). Returns True if sa40 is the suffix array."""
        import torch
        ok = C.c_int(0)
        stream = torch.cuda.current_stream(text.device).cuda_stream
        _native.check(self._lib.csa_verify_sa40_dev(self._h, text.data_ptr(), text.numel(), int(index_base),
                                                    sa40.data_ptr(), stream or None, C.byref(ok)))
        return bool(ok.value)


def pack_keys(text, key_words=1):
    """K-gram keys of every suffix of a uint16 device tensor: int64 tensor [n, key_words] (csa_pack_keys_u16_dev)."""
    import torch
    lib = _native.load()
    n = text.numel()
    keys = torch.empty((n, key_words), dtype=torch.int64, device=text.device)
    stream = torch.cuda.current_stream(text.device).cuda_stream
    _native.check(lib.csa_pack_keys_u16_dev(text.data_ptr(), n, int(key_words), keys.data_ptr(), stream or None))
    return keys


def partition_ids(text, pivots, p, n=None, text_len=None, want_ids=True, want_packed=True, want_sizes=True, sizes=None):
    """Partition id of every suffix against sorted pivots (csa_partition_ids_u16_dev; the reference's
    GPU_SACA::compute_partition_IDs, src/GPU_SACA.cu:854-1000, for a text chunk resident in HBM).
    text: uint16 device tensor; pivots: (p - 1, pivot_words) int64/uint64 device tensor, ascending.
    Returns (ids int16 tensor or None, packed int64 tensor or None, sizes int64 tensor or None); `sizes` is added to
    when given (chunked use)."""
    import torch
    lib = _native.load()
    assert text.is_cuda and text.element_size() == 2 and text.is_contiguous()
    n = text.numel() if n is None else int(n)
    text_len = text.numel() if text_len is None else int(text_len)
    assert pivots.dim() == 2, "pivots: one row of pivot_words 64-bit words per pivot"
    words = int(pivots.shape[1])
    assert pivots.element_size() == 8 and pivots.is_contiguous() and pivots.numel() == (p - 1) * words
    bits = int(lib.csa_partition_id_bits(p))
    dev = text.device
    ids = torch.empty(max(n, 1), dtype=torch.int16, device=dev) if want_ids else None
    packed = torch.zeros(((n + 63) // 64) * bits + 1, dtype=torch.int64, device=dev) if want_packed else None
    if want_sizes and sizes is None:
        sizes = torch.zeros(p, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    _native.check(lib.csa_partition_ids_u16_dev(text.data_ptr(), n, text_len, pivots.data_ptr() if pivots.numel() else None,
                                                words, int(p), ids.data_ptr() if want_ids else None,
                                                packed.data_ptr() if want_packed else None,
                                                sizes.data_ptr() if sizes is not None else None, stream or None))
    return (ids[:n] if want_ids else None), packed, sizes


def stage_slab(text, suf40, key_words, pid_map, p, ctx, generation0):
    """Keys (generation 0) and routing-tag pairs of a partition's suffixes, computed on the device from the text and the
    packed partition-id map (csa_stage_slab_u16_dev; the reference's host loop GPU_SACA::stage_slab,
    src/GPU_SACA.cu:1674-1691). suf40: uint8 tensor of 5-byte lanes. Returns (keys int64 [count, key_words] or None,
    beta int32 [count])."""
    import torch
    lib = _native.load()
    count = suf40.numel() // SA_WIDTH
    dev = text.device
    keys = torch.empty((max(count, 1), key_words), dtype=torch.int64, device=dev) if generation0 else None
    beta = torch.empty(max(count, 1), dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    _native.check(lib.csa_stage_slab_u16_dev(text.data_ptr(), text.numel(), suf40.data_ptr(), count, int(key_words),
                                             pid_map.data_ptr(), int(p), int(ctx), 1 if generation0 else 0,
                                             keys.data_ptr() if generation0 else None, beta.data_ptr(), stream or None))
    return (keys[:count] if generation0 else None), beta[:count]


def output_cut(lo, hi, chunk_bytes, c, chunk_c):
    """(piece_lo, piece_hi, head_lo, head_hi, tail_lo, tail_hi) of chunk c's share of the output byte range [lo, hi)
    (csa_output_cut; the reference's Output_File::cut, src/Output_File.cpp:18-35)."""
    out = (C.c_uint64 * 6)()
    _native.load().csa_output_cut(int(lo), int(hi), int(chunk_bytes), int(c), int(chunk_c), C.byref(out))
    return tuple(int(v) for v in out)


def sort_partition(text, key_words=1):
    """Host arrays in and out: uint16 numpy text -> uint8 numpy sa40 of 5*n bytes, plus statistics
    (csa_sort_partition_u16: device memory is allocated and released inside the call)."""
    lib = _native.load()
    text = np.ascontiguousarray(text, dtype=np.uint16)
    n = int(text.size)
    sa40 = np.zeros(SA_WIDTH * n, dtype=np.uint8)
    st = _native.CsaStats()
    _native.check(lib.csa_sort_partition_u16(text.ctypes.data if n else None, n, int(key_words),
                                             sa40.ctypes.data if n else None, C.byref(st)))
    return sa40, stats_to_dict(st)


def sort_partitions(texts, key_words=1, index_base=None, out=None):
    """Independent partitions in host memory, pipelined through the device (csa_sort_partitions_u16): the upload of one, the
    sort of another and the download of a third overlap. texts: uint16 numpy arrays (views of pinned memory transfer at the
    link's rate); out: optional uint8 numpy arrays of 5 * n bytes to fill. Returns (list of sa40 arrays, list of statistics)."""
    lib = _native.load()
    texts = [np.ascontiguousarray(t, dtype=np.uint16) for t in texts]
    count = len(texts)
    if out is None:
        out = [np.zeros(SA_WIDTH * t.size, dtype=np.uint8) for t in texts]
    assert len(out) == count and all(o.dtype == np.uint8 and o.size >= SA_WIDTH * t.size and o.flags["C_CONTIGUOUS"]
                                     for o, t in zip(out, texts))
    ptrs_in = (C.c_void_p * max(count, 1))(*[t.ctypes.data if t.size else None for t in texts])
    ptrs_out = (C.c_void_p * max(count, 1))(*[o.ctypes.data if t.size else None for o, t in zip(out, texts)])
    sizes = (C.c_uint64 * max(count, 1))(*[t.size for t in texts])
    bases = (C.c_uint64 * max(count, 1))(*[int(b) for b in index_base]) if index_base is not None else None
    stats = (_native.CsaStats * max(count, 1))()
    _native.check(lib.csa_sort_partitions_u16(count, ptrs_in, sizes, bases, int(key_words), ptrs_out, stats))
    return [o[:SA_WIDTH * t.size] for o, t in zip(out, texts)], [stats_to_dict(stats[k]) for k in range(count)]


class GPU_SACA:
    """`GPU_SACA(ip_path, op_path).build_SA()`: file of uint16 symbols in, file of 5-byte suffix indices out."""

    def __init__(self, ip_path, op_path, key_words=1):
        self.ip_path = ip_path
        self.op_path = op_path
        self.key_words = key_words
        self._timings = None

    def build_SA(self):
        text = np.fromfile(self.ip_path, dtype="<u2")
        sa40, stats = sort_partition(text, self.key_words)
        sa40.tofile(self.op_path)
        self._timings = stats
        return stats

    def timings(self):
        return self._timings
