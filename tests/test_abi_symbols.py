"""The C-ABI library loads without a GPU and exports every function that
include/pegahip.h declares; the Python prototypes cover the same set."""

import ctypes as C
import os
import re

import pytest

from pegaflow_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "pegahip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    names = re.findall(r"\b(pf_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_every_declared_symbol_is_exported():
    lib = C.CDLL(_lib.LIB_PATH)
    names = declared_functions()
    assert len(names) > 40
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_python_prototypes_cover_the_header():
    assert sorted(_lib.PROTOTYPES) == declared_functions()


def test_struct_sizes_match_the_header():
    assert C.sizeof(_lib.PfCopyDesc) == 48
    assert C.sizeof(_lib.PfKvLayout) == 72
    assert C.sizeof(_lib.PfHostMem) == 32


def test_no_device_is_an_error_not_a_fallback():
    """Without a HIP device every byte-moving entry point fails loudly."""
    lib = _lib.load()
    n = C.c_int()
    if lib.pf_device_count(C.byref(n)) == 0 and n.value > 0:
        return  # on a GPU box this check does not apply
    h = C.c_void_p()
    assert lib.pf_backend_create(_lib.PF_MODE_KERNEL, C.byref(h)) != 0
    assert lib.pf_last_error()
    mem = _lib.PfHostMem()
    assert lib.pf_host_alloc(4096, _lib.PF_HOST_HIP_ALLOC, -1, C.byref(mem)) != 0
    p = C.c_uint64()
    assert lib.pf_dev_malloc(4096, C.byref(p)) != 0


def test_header_is_plain_c(tmp_path):
    """include/pegahip.h is the boundary for C, C++ and FFI generators alike: it
    must compile as strict C99 and as C++11 with nothing else included."""
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for compiler, std, name in (("gcc", "-std=c99", "hdr.c"), ("g++", "-std=c++11", "hdr.cpp")):
        if shutil.which(compiler) is None:
            pytest.skip(f"{compiler} not installed")
        src = tmp_path / name
        src.write_text('#include "include/pegahip.h"\nint main(void) { return 0; }\n')
        proc = subprocess.run([compiler, std, "-Wall", "-Wextra", "-pedantic", "-Werror",
                               "-fsyntax-only", str(src), "-I", root], capture_output=True, text=True)
        assert proc.returncode == 0, proc.stderr
