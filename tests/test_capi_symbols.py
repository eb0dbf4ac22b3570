"""CPU checks of the C-ABI boundary: the shared library loads and exports every function
declared in include/grape_hip.h, and the Python signature table matches the header."""
import ctypes
import os
import re
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "grape_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(grape_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_functions():
    names = _declared()
    assert "grape_commit_i32" in names and "grape_fr_fold" in names and len(names) > 40


def test_library_exports_every_declared_symbol():
    from grape_amd import _capi
    if not os.path.exists(_capi.LIB_PATH):
        pytest.fail("libgrape_hip.so is not built: run `python -m grape_amd.build`")
    lib = ctypes.CDLL(_capi.LIB_PATH)
    missing = [n for n in _declared() if not hasattr(lib, n)]
    assert not missing, missing


def test_python_signatures_cover_header():
    from grape_amd import _capi
    assert sorted(_capi.SIGNATURES) == _declared()


def test_every_entry_point_cites_the_reference_or_says_why_not():
    text = open(HEADER).read()
    assert text.count("src/") > 20          # reference file:line citations


def test_product_does_not_touch_the_oracle():
    # nothing under grape_amd/ or include/ may import, link or load the CPU oracle
    bad = []
    for base in ("grape_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            for f in files:
                if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp", ".c")):
                    s = open(os.path.join(dirpath, f), errors="ignore").read()
                    if "grape_oracle" in s or "oracle/" in s or "import orc" in s:
                        bad.append(os.path.join(dirpath, f))
    assert not bad, bad
