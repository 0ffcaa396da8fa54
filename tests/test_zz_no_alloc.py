"""csa_radix_sort_pairs_static_dev: the entry point that allocates nothing (its scratch is a fixed array inside the
library, shared by all calls on a device and keeping the last call's contents), against csa_radix_sort_pairs_dev on the
same pairs, bit for bit, on calls in a row of shrinking size."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib

pytestmark = pytest.mark.gpu


def _dev(torch, a):
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a.view({8: np.int64, 4: np.int32}[a.dtype.itemsize])).cuda()


def test_sort_without_allocation_equals_the_sort_with_a_handle():
    import torch
    from cascade_amd import PartitionSorter, _native
    lib = _native.load()
    assert torch.cuda.is_available()
    rng = np.random.default_rng(12)
    limit = 1 << 20  # CSA_STATIC_SORT_MAX_PAIRS
    stream = torch.cuda.current_stream().cuda_stream
    with PartitionSorter(limit) as s:
        # the largest size first, then smaller ones: what a call leaves in the scratch must not reach the next call
        for n, b, e, skew in ((limit, 0, 64, 0), (300001, 0, 64, 0), (8193, 3, 37, 0), (777, 0, 64, 50), (1, 0, 64, 0),
                              (limit - 5, 16, 48, 20)):
            keys = rng.integers(0, 1 << 63, n, dtype=np.uint64) >> np.uint64(skew)
            vals = rng.permutation(n).astype(np.uint32)
            print(f"  static sort n={n} bits=[{b},{e})", flush=True)
            k0, v0 = _dev(torch, keys), _dev(torch, vals)
            s.radix_sort_pairs(k0, v0, b, e)
            k1, v1 = _dev(torch, keys), _dev(torch, vals)
            free_before = torch.cuda.mem_get_info()[0]
            _native.check(lib.csa_radix_sort_pairs_static_dev(k1.data_ptr(), v1.data_ptr(), n, b, e, stream or None))
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before  # nothing was allocated on the device
            assert torch.equal(k1, k0) and torch.equal(v1, v0), (n, b, e)
            if n <= 300001:
                wk, wv = oracle_lib.stable_sort_pairs(keys, vals, b, e)
                assert np.array_equal(k1.cpu().numpy().view(np.uint64), wk) and np.array_equal(v1.cpu().numpy().view(np.uint32), wv)
    # beyond the fixed scratch: refused with a clear error, nothing launched
    k = torch.zeros(limit + 1, dtype=torch.int64, device="cuda")
    v = torch.zeros(limit + 1, dtype=torch.int32, device="cuda")
    rc = lib.csa_radix_sort_pairs_static_dev(k.data_ptr(), v.data_ptr(), limit + 1, 0, 64, None)
    assert rc == _native.CSA_ERR_TOO_LARGE and b"exceed" in lib.csa_last_error()
