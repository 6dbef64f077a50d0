"""Host-side checks that need no GPU: the C-ABI library loads, exports exactly what the header
declares, and rejects bad arguments with status codes before touching the device."""
import ctypes as C
import os
import re

import pytest

from conftest import ROOT

import permutohedral_lattice_amd as pla


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "permutohedral_lattice.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pl_[a-z_0-9]+)\s*\(", text)))


def test_library_is_in_tree_and_exports_every_declared_symbol():
    assert os.path.dirname(pla.LIB_PATH) == os.path.join(ROOT, "permutohedral_lattice_amd")
    declared = _declared_functions()
    assert declared == sorted(pla.EXPORTS)
    lib = C.CDLL(pla.LIB_PATH)
    for name in declared:
        assert getattr(lib, name) is not None


def test_supported_dimensions():
    for pd in range(1, 9):
        for vd in (2, 3, 4, 5, 8, 9, 22, 64):
            assert pla.supported(pd, vd)
    assert not pla.supported(0, 4)
    assert not pla.supported(9, 4)
    assert not pla.supported(5, 1)


def test_strerror_covers_every_status():
    seen = set()
    for code in range(0, -8, -1):
        msg = pla._lib.pl_strerror(code).decode()
        assert msg and msg != "unknown status"
        seen.add(msg)
    assert len(seen) == 8
    assert pla._lib.pl_strerror(-99).decode() == "unknown status"


@pytest.mark.parametrize("pd,vd,n,expect", [
    (5, 4, -1, pla.PL_EINVAL),
    (0, 4, 10, pla.PL_EINVAL),
    (5, 1, 10, pla.PL_EINVAL),
    (9, 4, 10, pla.PL_EUNSUPPORTED),
    (5, 4, 2 ** 30, pla.PL_EOVERFLOW),      # N*(pd+1) replay rows beyond the supported range
])
def test_create_rejects_bad_arguments_without_a_device(pd, vd, n, expect):
    h = C.c_void_p()
    assert pla._lib.pl_create(pd, vd, n, None, None, C.byref(h)) == expect
    assert not h.value
    assert pla._lib.pl_create(5, 4, 10, None, None, None) == pla.PL_EINVAL


def test_null_handles_are_rejected():
    lib = pla._lib
    assert lib.pl_filter(None, None, None, None, 0) == pla.PL_EINVAL
    assert lib.pl_build(None, None) == pla.PL_EINVAL
    assert lib.pl_apply(None, None, None, 0) == pla.PL_EINVAL
    dims = (C.c_int * 2)(8, 8)
    assert lib.pl_filter_image(None, None, None, None, 3, 2, dims, 1.0, 1.0, 0) == pla.PL_EINVAL
    assert lib.pl_build_image(None, None, 3, 2, dims, 1.0, 1.0) == pla.PL_EINVAL
    assert lib.pl_num_vertices(None, None) == pla.PL_EINVAL
    assert lib.pl_set_option(None, 1, 0) == pla.PL_EINVAL
    assert lib.pl_destroy(None) == pla.PL_OK


def test_op_and_feature_builder_argument_checks():
    lib = pla._lib
    dims = (C.c_int * 2)(8, 8)
    bad = (C.c_int * 2)(8, 0)
    # no spatial dims / no channels / non-positive extent
    assert lib.pl_lattice_filter_op(None, None, None, 1, 0, dims, 3, 3, 1, 1.0, 1.0, 1.0, 0, None, None) == pla.PL_EINVAL
    assert lib.pl_lattice_filter_op(None, None, None, 1, 2, dims, 0, 3, 1, 1.0, 1.0, 1.0, 0, None, None) == pla.PL_EINVAL
    assert lib.pl_lattice_filter_op(None, None, None, 1, 2, bad, 3, 3, 1, 1.0, 1.0, 1.0, 0, None, None) == pla.PL_EINVAL
    # bilateral without a reference image
    assert lib.pl_lattice_filter_op(None, None, None, 1, 2, dims, 3, 3, 1, 1.0, 1.0, 1.0, 0, None, None) == pla.PL_EINVAL
    # pd = 2 + 7 reference channels is not instantiated
    assert lib.pl_lattice_filter_op(None, None, None, 0, 2, dims, 3, 7, 1, 1.0, 1.0, 1.0, 0, None, None) == pla.PL_EUNSUPPORTED
    # more than INT32_MAX tensor elements, as the reference op refuses
    big = (C.c_int * 2)(65536, 32768)
    assert lib.pl_lattice_filter_op(None, None, None, 1, 2, big, 3, 3, 1, 1.0, 1.0, 1.0, 0, None, None) == pla.PL_EOVERFLOW
    # empty batch is a no-op
    assert lib.pl_lattice_filter_op(None, None, None, 0, 2, dims, 3, 3, 1, 1.0, 1.0, 1.0, 0, None, None) == pla.PL_OK
    assert lib.pl_compute_positions(None, None, -1, 3, 2, dims, 1.0, 1.0, None) == pla.PL_EINVAL
    assert lib.pl_compute_positions(None, None, 0, 3, 2, dims, 1.0, 1.0, None) == pla.PL_OK
    assert lib.pl_compute_positions(None, None, 64, 3, 2, dims, 1.0, 1.0, None) == pla.PL_EINVAL


def test_python_constants_are_the_headers():
    """Every PL_* enumerator of the header has the same value in the Python mirror."""
    text = open(os.path.join(ROOT, "include", "permutohedral_lattice.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    found = {name: int(value) for name, value in re.findall(r"\b(PL_[A-Z_0-9]+)\s*=\s*(-?\d+)", text)}
    assert len(found) >= 20
    for name, value in found.items():
        assert getattr(pla, name) == value, name


def _stub_library(tmp_path, layout_version, row_bytes):
    """A library with every export of the real one, all doing nothing, that reports the given
    array layout: what a build of the kernels with another replay-row format would look like to
    the loader."""
    import subprocess
    src = ["int pl_library_info(int what, long long *value) {",
           "    *value = what == 1 ? %d : (what == 2 ? %d : 0);" % (layout_version, row_bytes),
           "    return 0;", "}"]
    for name in pla.EXPORTS:
        if name == "pl_library_info":
            continue
        if name == "pl_strerror":
            src.append('const char *pl_strerror(int s) { (void)s; return "stub"; }')
        else:
            src.append("int %s(void) { return 0; }" % name)
    c_file = tmp_path / "stub.c"
    c_file.write_text("\n".join(src) + "\n")
    so = tmp_path / ("libstub_%d_%d.so" % (layout_version, row_bytes))
    subprocess.run(["gcc", "-shared", "-fPIC", "-o", str(so), str(c_file)], check=True)
    return str(so)


def test_library_reports_the_layout_the_python_side_drives():
    assert pla.LAYOUT_VERSION == pla._library_property(pla._lib, pla.PL_LIB_LAYOUT_VERSION)
    assert pla.REPLAY_ROW_BYTES == pla._library_property(pla._lib, pla.PL_LIB_REPLAY_ROW_BYTES)
    text = open(os.path.join(ROOT, "include", "permutohedral_lattice.h")).read()
    assert int(re.search(r"#define PL_LAYOUT_VERSION (\d+)", text).group(1)) == pla.LAYOUT_VERSION
    v = C.c_longlong()
    assert pla._lib.pl_library_info(99, C.byref(v)) == pla.PL_EINVAL
    assert pla._lib.pl_library_info(1, None) == pla.PL_EINVAL


def test_library_source_hash_is_that_of_the_sources_in_the_tree():
    from permutohedral_lattice_amd import build
    assert pla.library_source_hash() == build.source_hash(), \
        "the library in the tree was built from other sources: run permutohedral_lattice_amd/build.py"


def test_a_library_with_another_array_layout_is_refused(tmp_path):
    # same layout: loads
    pla._load(_stub_library(tmp_path, pla.LAYOUT_VERSION, pla.REPLAY_ROW_BYTES))
    # replay rows of 6 bytes, or another layout version: refused before anything is bound
    with pytest.raises(ImportError, match="array layout version"):
        pla._load(_stub_library(tmp_path, pla.LAYOUT_VERSION, 6))
    with pytest.raises(ImportError, match="array layout version"):
        pla._load(_stub_library(tmp_path, pla.LAYOUT_VERSION + 1, pla.REPLAY_ROW_BYTES))


def test_documented_build_command_lists_every_source():
    from permutohedral_lattice_amd import build
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    for path in build.SOURCES:
        assert os.path.relpath(path, ROOT) in text, path
