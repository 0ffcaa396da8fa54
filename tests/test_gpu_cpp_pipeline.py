"""The C++ mirror of the reference's builder class (include/cascade_gpu_saca.hpp) driven from C++, as Cascade's dispatcher
drives its own class: tests/cpp/slab_pipeline.cpp (built by cascade_amd/build.py) builds the suffix array of a
multi-partition text through sort_and_init_rank_and_filter / sort_and_re_rank_and_filter / scatter_to_rank_order on
Partition_Assemblies of pinned Staging_Slabs. The program compares its result with the resident single-partition sort; here
the file it writes is also compared with the CPU oracle's suffix array."""
import os
import subprocess

import numpy as np
import pytest

import oracle_lib

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "slab_pipeline")


@pytest.mark.parametrize("n,p,key_words,chunk_cap,sigma", [(100000, 7, 1, 4096, 4), (150000, 16, 4, 8192, 3), (60000, 1, 2, 32768, 2),
                                                           (200000, 40, 1, 4096, 300)])
def test_cpp_builder_members_on_host_slabs_build_the_oracles_suffix_array(tmp_path, n, p, key_words, chunk_cap, sigma):
    assert os.path.exists(EXE), "tests/cpp/slab_pipeline is not built (python -m cascade_amd.build)"
    out = tmp_path / "sa40"
    print(f"  slab_pipeline n={n} p={p} key_words={key_words} chunk_cap={chunk_cap} sigma={sigma}", flush=True)
    run = subprocess.run([EXE, str(n), str(p), str(key_words), str(chunk_cap), str(1000 + p), str(sigma), str(out)], capture_output=True,
                         text=True, timeout=300)
    assert run.returncode == 0, (run.stdout, run.stderr)
    assert run.stdout.startswith("OK "), run.stdout
    generations = int(run.stdout.split("generations=")[1].split()[0])
    assert generations >= 8  # the planted repeat keeps suffixes tied for many generations
    T = np.fromfile(str(out) + ".text", dtype=np.uint16)
    got = np.fromfile(out, dtype=np.uint8)
    want = oracle_lib.u64_to_sa40(oracle_lib.prefix_doubling(T, 1)[0])[:5 * n]  # (the long repeat rules out the comparison sort)
    assert T.size == n and np.array_equal(got, want)
