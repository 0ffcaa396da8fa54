"""The benchmark configurations at their full sizes, through the C ABI. The headline configuration (1e9 tokens), sorted with
the tile order the headline figure is measured with, is judged by the CPU oracle's O(n) verifier (the reference's rule of
test/end-to-end.cpp:46-80: a permutation whose every adjacent pair is in order; the suffix array is unique, so passing it
is byte-equality with the reference's sort). All configurations are also checked by properties that need no host pass:
the device verifier accepts the result and rejects it after one swap; the entries sum to n (n - 1) / 2; the number of
generations and the active counts are those of a second, independent run."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.timeout(600)
@pytest.mark.parametrize("config,exclusive,oracle_verifier", [(2, False, True), (3, False, False), (3, True, True), (5, True, True),
                                                              (4, True, True)],
                         ids=["C2-arrival-oracle", "C3-arrival", "C3-xcd_chunked-oracle", "C5-xcd_chunked-oracle", "C4-xcd_chunked-oracle"])
def test_full_size_configuration_sorts_to_a_verified_suffix_array(config, exclusive, oracle_verifier):
    import torch
    import oracle_lib
    from cascade_amd import PartitionSorter, workloads
    n = workloads.default_n(config)
    print(f"  full size C{config} n={n}", flush=True)
    T = workloads.generate(config, n)
    d_text = torch.from_numpy(T.view(np.int16)).cuda()
    if not oracle_verifier:
        del T
    # exclusive: the XCD-chunked tile order of the radix passes (the test is the only user of the device)
    s = PartitionSorter(n, key_words=1, device_exclusive=exclusive)
    try:
        out = s.sort(d_text)
        stats = s.last_stats
        if oracle_verifier:  # about 23 bytes of host memory per suffix
            print("  oracle verifier on the host", flush=True)
            assert oracle_lib.is_correct_sa40(out.cpu().numpy(), T)
            del T
        assert s.verify(d_text, out)
        # permutation by another route: 40-bit entries, little-endian, sum = n (n - 1) / 2
        b = out.view(n, 5).to(torch.int64)
        total = int(b[:, 0].sum()) + (int(b[:, 1].sum()) << 8) + (int(b[:, 2].sum()) << 16) + (int(b[:, 3].sum()) << 24) + (
            int(b[:, 4].sum()) << 32)
        del b
        assert total == n * (n - 1) // 2
        # one swap of two neighbouring entries (distinct suffixes, so the order breaks) must be caught
        r = n // 3
        e0, e1 = out[5 * r:5 * r + 5].clone(), out[5 * r + 5:5 * r + 10].clone()
        out[5 * r:5 * r + 5], out[5 * r + 5:5 * r + 10] = e1, e0
        assert not s.verify(d_text, out)
        out2 = s.sort(d_text)
        assert s.last_stats["active"] == stats["active"] and s.last_stats["generations"] == stats["generations"]
        assert s.verify(d_text, out2)
    finally:
        s.close()


@pytest.mark.timeout(600)
def test_largest_partition_at_the_largest_index_base():
    """n = 2^31 - 1 suffixes (MAX_PART_SZ, include/bit-layout.hpp:63-68) ending at suffix index 2^40 - 1, the last
    one a 5-byte entry can hold (include/sa40.hpp:72-75): uniform random symbols, generated on the device. The suffix array
    from index 0 goes through the oracle's verifier on the host; the one at the largest base must be that array shifted."""
    import torch
    from cascade_amd import PartitionSorter
    n = (1 << 31) - 1
    base = (1 << 40) - n
    print(f"  largest partition n={n} index_base={base}", flush=True)
    g = torch.Generator(device="cuda")
    g.manual_seed(20240531)
    d_text = torch.randint(-32768, 32768, (n,), dtype=torch.int16, device="cuda", generator=g)
    s = PartitionSorter(n, key_words=1)
    try:
        # the same partition from index 0 is judged by the CPU oracle's O(n) verifier (the reference's rule,
        # test/end-to-end.cpp:46-80; about 23 bytes of host memory per suffix, 49 GB here)
        import oracle_lib
        out0 = s.sort(d_text)
        print("  oracle verifier on the host", flush=True)
        assert oracle_lib.is_correct_sa40(out0.cpu().numpy(), d_text.cpu().numpy().view(np.uint16))
        out = s.sort(d_text, index_base=base)
        # ... and at the largest base every entry is the verified one plus the base (compared in pieces of 2^26 entries)

        def entries(lanes):
            e = lanes[:, 0].to(torch.int64)
            for k in range(1, 5):
                e |= lanes[:, k].to(torch.int64) << (8 * k)
            return e
        for lo in range(0, n, 1 << 26):
            hi = min(n, lo + (1 << 26))
            assert bool((entries(out.view(n, 5)[lo:hi]) == entries(out0.view(n, 5)[lo:hi]) + base).all()), lo
        del out0
        assert s.last_stats["n"] == n and s.last_stats["generations"] >= 1
        assert s.verify(d_text, out, index_base=base)
        assert not s.verify(d_text, out, index_base=base - 1)
        lanes = out.view(n, 5)
        total = sum(int(lanes[:, k].sum(dtype=torch.int64)) << (8 * k) for k in range(5))
        assert total == n * (n - 1) // 2 + n * base
        # the largest entry is 2^40 - 1: all five bytes 0xFF somewhere in the output
        assert bool((lanes == 255).all(dim=1).any())
    finally:
        s.close()


@pytest.mark.timeout(300)
def test_three_dispatcher_threads_sorting_large_texts_at_once():
    """Three threads, each with its own handle and stream, sort texts of 2^25 symbols at the same time
    (the reference's three buffer sets, include/GPU_SACA.hpp:90-91, src/GPU_SACA.cu:1539-1589). Thousands of tiles
    of three radix passes then compete for the device: with the default tile order (by arrival) every wait of a
    pass ends, whatever the other launches hold."""
    import threading
    import torch
    from cascade_amd import PartitionSorter, workloads
    n, per_thread = 1 << 25, 3
    T = workloads.generate(3, 3 * per_thread * n)
    h_text = torch.from_numpy(T.view(np.int16)).reshape(3 * per_thread, n).pin_memory()
    del T
    outs = [None] * (3 * per_thread)
    errors = []

    def dispatcher(t):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream), PartitionSorter(n) as s:
                for q in range(t, 3 * per_thread, 3):
                    d = h_text[q].cuda(non_blocking=True)
                    outs[q] = s.sort(d).clone()
                    stream.synchronize()
        except Exception as e:  # noqa: BLE001 - reported below, in the main thread
            errors.append((t, repr(e)))

    print("  three dispatcher threads, 2^25 symbols each", flush=True)
    threads = [threading.Thread(target=dispatcher, args=(t,)) for t in range(3)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    assert not errors, errors
    with PartitionSorter(n) as s:
        for q in range(3 * per_thread):
            assert s.verify(h_text[q].cuda(), outs[q]), q
