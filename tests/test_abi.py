"""The C-ABI library loads and exports exactly what include/cascade_hip.h declares. No GPU needed."""
import ctypes as C
import os
import re

import pytest

from cascade_amd import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    src = open(os.path.join(ROOT, "include", "cascade_hip.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(csa_[a-z0-9_]+)\s*\(", src)))


def test_header_and_binding_agree():
    assert declared_functions() == sorted(_native.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = _native.load()
    for name in declared_functions():
        assert hasattr(lib, name), name


def test_struct_layouts_match_the_header(tmp_path):
    """The ctypes structures have the sizes and field offsets the C compiler gives the header's structs."""
    import subprocess
    src = tmp_path / "layout.c"
    src.write_text('''#include <stddef.h>
#include <stdio.h>
#include "cascade_hip.h"
int main(void) {
    printf("%zu %zu %zu %zu\\n", sizeof(csa_stats), offsetof(csa_stats, ms), offsetof(csa_stats, radix_ms), offsetof(csa_stats, presorted));
    printf("%zu %zu\\n", sizeof(csa_step_result), offsetof(csa_step_result, incoherent_pills));
    printf("%zu %zu %zu\\n", sizeof(csa_slab), offsetof(csa_slab, off), offsetof(csa_slab, outbox_sz));
    return 0;
}
''')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), "-o", str(exe), str(src)], check=True)
    lines = subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split("\n")
    st, sr, sl = _native.CsaStats, _native.CsaStepResult, _native.CsaSlab
    assert [int(v) for v in lines[0].split()] == [C.sizeof(st), st.ms.offset, st.radix_ms.offset, st.presorted.offset]
    assert [int(v) for v in lines[1].split()] == [C.sizeof(sr), sr.incoherent_pills.offset]
    assert [int(v) for v in lines[2].split()] == [C.sizeof(sl), sl.off.offset, sl.outbox_sz.offset]


def test_argument_errors_need_no_gpu():
    lib = _native.load()
    assert lib.csa_bytes_per_suffix(1) == 60
    h = C.c_void_p()
    assert lib.csa_create(10, 5, C.byref(h)) == _native.CSA_ERR_ARG
    assert b"key_words" in lib.csa_last_error()
    assert lib.csa_create(1 << 31, 1, C.byref(h)) == _native.CSA_ERR_TOO_LARGE
    assert lib.csa_sort_partition_u16(None, 1 << 31, 1, None, None) == _native.CSA_ERR_TOO_LARGE
    assert lib.csa_sort_partition_u16_dev(None, None, 0, 0, None, None, 0, None) == _native.CSA_ERR_ARG
    with pytest.raises(_native.CascadeError):
        _native.check(lib.csa_radix_sort_pairs_dev(None, None, None, 0, 0, 64, None))


def test_builder_mirror_compiles_as_plain_cpp_and_the_program_is_built():
    """include/cascade_gpu_saca.hpp (the reference's builder surface over the C ABI) needs no HIP header, and
    cascade_amd/cascade_sa, the command-line builder made from it, refuses a call without arguments as the reference's
    program does (src/main.cu:15-19)."""
    import subprocess
    hdr = os.path.join(ROOT, "include", "cascade_gpu_saca.hpp")
    subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Wextra", "-Werror", "-x", "c++", hdr], check=True)
    exe = os.path.join(ROOT, "cascade_amd", "cascade_sa")
    assert os.path.exists(exe), "run python -m cascade_amd.build"
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 1 and "Usage:" in r.stderr
