"""The C-ABI library loads without a GPU and exports every entry point that
include/tandem_hip.h declares (no compute calls here)."""

import ctypes
import os
import re

from helpers import GOLDEN

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "tandem_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tdm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_entry_point():
    from tandem_amd import _lib

    L = _lib.lib()
    names = declared_functions()
    assert len(names) >= 11
    for name in names:
        assert hasattr(L, name), f"{name} is declared in tandem_hip.h but not exported"
    assert sorted(_lib.exported_symbols()) == names, "the ctypes binding and the header disagree"
    assert L.tdm_abi_version() == _lib.ABI_VERSION
    assert isinstance(L.tdm_last_error(), bytes)  # the last failed call's message on this thread (empty before any)


def test_struct_layouts_match_the_header():
    from tandem_amd import _lib

    assert ctypes.sizeof(_lib.Pair) == 24
    assert ctypes.sizeof(_lib.FoldSeg) == 8 * 8 * 2 + 16
    assert ctypes.sizeof(_lib.AdamwScalars) == 36


def test_argument_errors_need_no_gpu():
    from tandem_amd import _lib

    L = _lib.lib()
    assert L.tdm_k1_reduce_step(None, 17, 0, 2, 1, 1, 0, None) == 1
    assert b"npairs" in L.tdm_last_error()
    assert L.tdm_k1_copy_step(None, 0, 99, 0, None) == 1
    segs = (_lib.FoldSeg * 2)()
    segs[0].count, segs[1].count = 5, 5000
    assert L.tdm_k2_table_bytes(segs, 0, 0) > 0 and L.tdm_k2_table_bytes(segs, 2, 0) > L.tdm_k2_table_bytes(segs, 1, 0)
    assert L.tdm_k2_table_bytes(segs, 2, 99) == -1
    assert L.tdm_set_blocks_per_cu(50_000) == 1
    assert L.tdm_set_blocks_per_cu(0) == 0
    assert L.tdm_set_xcd_group(6, 0) == 1 and b"family" in L.tdm_last_error()
    assert L.tdm_set_xcd_group(0, 13) == 1 and b"shift" in L.tdm_last_error()
    assert L.tdm_set_xcd_group(3, 4) == 0 and L.tdm_set_xcd_group(-1, -1) == 0
    assert L.tdm_set_ring_form(2) == 1 and b"ring form" in L.tdm_last_error()
    assert L.tdm_set_ring_form(1) == 0 and L.tdm_set_ring_form(-1) == 0
    assert L.tdm_set_occupancy_pad(4, 65537) == 1 and L.tdm_set_occupancy_pad(4, 8192) == 0 and L.tdm_set_occupancy_pad(-1, -1) == 0
    a, b, c = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    assert L.tdm_build_geometry(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)) == 0
    assert (a.value, b.value, c.value) == (4096, 128, 4096) and c.value == L.tdm_table_tile_bytes()
    assert L.tdm_build_geometry(None, ctypes.byref(b), ctypes.byref(c)) == 1
    assert L.tdm_k2_static_max_tiles() == 16384
    # the static bucket fold checks its arguments before it touches the GPU
    assert L.tdm_k2_bucket_fold_static(segs, 2, 2, 99, 1, 0, None) == 1 and b"dtype" in L.tdm_last_error()
    assert L.tdm_k2_bucket_fold_static(segs, 2, 9, 0, 1, 0, None) == 1 and b"world" in L.tdm_last_error()


def test_the_measurement_probe_is_a_library_of_its_own():
    """The stream-mix probe is not part of the plug-in: libtandem_hip.so does not export it, its header
    does not declare it, and libtandem_probe.so exports what include/tandem_probe.h declares and
    checks its arguments without a GPU."""
    import subprocess

    from tandem_amd import _lib, _probe

    assert not hasattr(_lib.lib(), "tdm_probe_stream_mix")
    assert not [n for n in declared_functions() if "probe" in n]
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "tandem_probe.h")).read(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(tdm_[a-z0-9_]+)\s*\(", text)))
    assert declared == ["tdm_probe_last_error", "tdm_probe_stream_mix"]
    P = _probe.lib()
    assert P.tdm_probe_stream_mix(None, 0, None, 0, 16, 1, 0, 0, None) == 1 and b"streams" in P.tdm_probe_last_error()
    out = subprocess.run(["nm", "-D", "--defined-only", _probe.PROBE_PATH], stdout=subprocess.PIPE, text=True, check=True).stdout
    assert sorted(l.split()[-1] for l in out.splitlines() if l.split()[-1].startswith("tdm_")) == declared
    res = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c",
                          os.path.join(ROOT, "include", "tandem_probe.h")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from tandem_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    try:
        _lib.lib()
    except _lib.HipLibraryMissing as e:
        assert "no CPU" in str(e)
    else:
        raise AssertionError("a missing library must raise")


def test_cpu_tensors_are_refused():
    import pytest
    import torch

    from tandem_amd import LocalWorld, ShardedAdamW

    with pytest.raises(ValueError, match="no CPU path"):
        LocalWorld(2).all_reduce([torch.zeros(4), torch.zeros(4)])
    with pytest.raises(ValueError, match="no CPU path"):
        ShardedAdamW().update("k", torch.zeros(4), torch.zeros(4))


def test_fixtures_present():
    for f in ("ring_w2.npz", "ring_w3.npz", "ring_w4.npz", "ring_dtypes_w3.npz", "adamw.npz", "plans.json", "data.json"):
        assert os.path.exists(os.path.join(GOLDEN, f))


def test_the_header_is_plain_c():
    """include/tandem_hip.h is what a C, Go (cgo) or Rust (bindgen) host would bind: it must compile as C99 on its own."""
    import shutil
    import subprocess

    import pytest

    if shutil.which("gcc") is None:
        pytest.skip("needs gcc")
    header = os.path.join(ROOT, "include", "tandem_hip.h")
    res = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c", header],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout


def test_the_library_exports_only_what_the_header_declares():
    """Built with hidden visibility: apart from weak instantiations of the C++ standard library's templates, the
    dynamic symbol table holds the header's entry points and nothing of the library's own C++."""
    import shutil
    import subprocess

    import pytest

    from tandem_amd import _lib

    if shutil.which("nm") is None or not os.path.exists(_lib.LIB_PATH):
        pytest.skip("needs nm and the built library")
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], stdout=subprocess.PIPE, text=True, check=True).stdout
    names = [line.split()[-1] for line in out.splitlines() if line.strip()]
    ours = sorted(n for n in names if n.startswith("tdm_"))
    assert ours == _lib.exported_symbols()
    assert not [n for n in names if "tandem_hip" in n], "internal C++ symbols are exported"


def test_the_product_stays_clear_of_the_checkers():
    """Nothing the package is made of names the oracle or the test doubles: the library is built from
    tandem_amd/csrc alone, and no Python module of the package imports from oracle/ or tests/."""
    import re

    from tandem_amd import build

    pkg = os.path.join(ROOT, "tandem_amd")
    assert all(os.path.dirname(os.path.join(build.CSRC, s)) == build.CSRC for s in build.SOURCES + build.PROBE_SOURCES)
    assert "probe.hip" not in build.SOURCES
    for dirpath, _, names in os.walk(pkg):
        for name in names:
            if not name.endswith((".py", ".hip", ".h")):
                continue
            text = open(os.path.join(dirpath, name)).read()
            assert not re.search(r"^\s*(from|import)\s+(oracle|tests)\b", text, re.M), name
            assert "fake_hip" not in text and "fake_kernels" not in text and "oracle/" not in text, name
