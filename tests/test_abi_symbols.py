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


def header_structs():
    """{struct name: [field names]} of every `typedef struct pf_x { ... } pf_x;`."""
    text = open(os.path.join(ROOT, "include", "pegahip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for name, body in re.findall(r"typedef struct (pf_\w+) \{(.*?)\} \1;", text, flags=re.S):
        fields = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            # `a, b, c` after one type (pf_save_profile) or a single declarator
            for part in decl.split(","):
                fields.append(re.findall(r"(\w+)\s*(?:\[\d+\])?\s*$", part.strip())[0])
        out[name] = fields
    return out


@pytest.fixture(scope="module")
def c_layout(tmp_path_factory):
    """Sizes and field offsets as a C compiler lays the header out: the output of
    tests/native/abi_layout.c, which also pins every number with _Static_assert."""
    import json
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("gcc not installed")
    exe = tmp_path_factory.mktemp("abi") / "abi_layout"
    proc = subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", ROOT,
                           os.path.join(ROOT, "tests", "native", "abi_layout.c"), "-o", str(exe)],
                          capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
    return json.loads(subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout)


def test_c_layout_covers_every_struct_and_field_of_the_header(c_layout):
    structs = header_structs()
    assert len(structs) >= 20
    assert sorted(c_layout) == sorted(structs)
    for name, fields in structs.items():
        assert list(c_layout[name]["fields"]) == fields, name


def test_ctypes_mirrors_match_the_c_layout(c_layout):
    """Every struct of the header has a ctypes mirror with the same size, the same
    fields in the same order and every field at the same offset (a swapped pair
    of equally sized fields changes the names at the offsets)."""
    for name, layout in c_layout.items():
        mirror = getattr(_lib, "".join(part.capitalize() for part in name.split("_")), None)
        assert mirror is not None, f"pegaflow_amd/_lib.py has no mirror of {name}"
        assert C.sizeof(mirror) == layout["size"], name
        assert [f[0] for f in mirror._fields_] == list(layout["fields"]), name
        for field, offset in layout["fields"].items():
            assert getattr(mirror, field).offset == offset, f"{name}.{field}"


def test_copy_desc_is_the_reference_field_order(c_layout):
    # transfer/mod.rs:36-44: device, host, host_device, size, device_allocation, host_allocation
    assert list(c_layout["pf_copy_desc"]["fields"]) == [
        "device", "host", "host_device", "size", "device_allocation", "host_allocation"]
    assert c_layout["pf_copy_desc"]["size"] == 48


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
