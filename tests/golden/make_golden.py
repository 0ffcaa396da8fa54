"""Writes tests/golden/fixtures.npz and tests/golden/c1_sha256.txt.

The expected suffix arrays come from the reference's own CPU sort (test/query.cpp:42-55, build_sa40), compiled
from its sources by oracle/Makefile into oracle/_ref/libcascade_ref.so. Run in the container that holds
/root/reference:   make -C oracle && python tests/golden/make_golden.py
The fixtures are data only: input symbols and the sa40 bytes the reference produced for them.
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle_lib  # noqa: E402
import texts  # noqa: E402
from cascade_amd import workloads  # noqa: E402


def main():
    ref = oracle_lib.ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libcascade_ref.so is missing: run `make -C oracle` where /root/reference exists")
    arrays = {}
    for name, T in texts.fixture_suite():
        arrays[f"{name}.text"] = T
        arrays[f"{name}.sa40"] = oracle_lib.build_sa40(T, lib=ref)
    np.savez_compressed(os.path.join(HERE, "fixtures.npz"), **arrays)
    c1 = workloads.generate(1)
    sa = oracle_lib.build_sa40(c1, lib=ref)
    with open(os.path.join(HERE, "c1_sha256.txt"), "w") as f:
        f.write(f"text {hashlib.sha256(c1.tobytes()).hexdigest()}\n")
        f.write(f"sa40 {hashlib.sha256(sa.tobytes()).hexdigest()}\n")
    print(f"wrote {len(arrays) // 2} fixtures and the C1 digests")


if __name__ == "__main__":
    main()
