"""Host walk over the address arithmetic of the wide-table commitment kernels (the expressions of
grape_amd/csrc/commit_geometry.hpp, shared by the kernels, their launcher and this build): for each
shape every wave's scalar reads, table gathers, partial-sum stores and loads and output rows stay
inside their buffers and every grid inside the limits of a launch.  The shapes include the one
commitment that once ended in an illegal access on the GPU ((2^20 + 3) rows of 4096 int32 scalars,
then still one launch with a 17 GB buffer of partial sums) - its arithmetic holds, in that layout and
in slabs - the largest size a call accepts (2^28 scalars) and the long-row shapes of the layer driver."""
import ctypes
import os
import subprocess
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "native", "commit_geometry_host.cpp")
LIB = os.path.join(HERE, "native", "libcommit_geometry_host.so")
HDR = os.path.join(HERE, "..", "grape_amd", "csrc", "commit_geometry.hpp")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB) or any(os.path.getmtime(d) > os.path.getmtime(LIB) for d in (SRC, HDR)):
        subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-unknown-pragmas", "-o", LIB, SRC])
    l = ctypes.CDLL(LIB)
    l.commit_geometry_check.restype = ctypes.c_longlong
    l.commit_geometry_check.argtypes = [ctypes.c_size_t, ctypes.c_uint32, ctypes.c_size_t, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                        ctypes.c_size_t, ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(ctypes.c_size_t),
                                        ctypes.POINTER(ctypes.c_size_t), ctypes.c_char_p, ctypes.c_size_t]
    return l


def _walk(lib, rows, rowlen, N, nw, K, elem_words, slab_segments=32768):
    pb, nl = ctypes.c_size_t(0), ctypes.c_size_t(0)
    rep = ctypes.create_string_buffer(256)
    bad = lib.commit_geometry_check(rows * rowlen, rowlen, N, nw, K, elem_words, slab_segments, 32, 24, ctypes.byref(pb), ctypes.byref(nl), rep, 256)
    return bad, pb.value, nl.value, rep.value.decode()


SHAPES = [
    # rows, rowlen, generators, windows, digit values, words per scalar
    (4096, 4096, 4096, 1, 32768, 1),          # configs[1]
    (32768, 4096, 4096, 19, 8192, 8),         # 2^27 full-width scalars (the exp lookup of the layer)
    (65536, 4096, 4096, 1, 32768, 1),         # 2^28 scalars: the largest call
    (8192, 4096, 4096, 19, 8192, 8),          # 2^25 full-width
    (40000, 8, 8, 1, 32768, 1),               # many short rows, two slabs
    (1, 65536, 65536, 26, 512, 8),            # one long row in 64-lane segments
    (3, 262144, 262144, 2, 256, 1),           # the layer driver's 262 144-column rows, two-digit table
    (700, 100, 128, 5, 128, 1),               # ragged: row length no multiple of 64
    ((1 << 20) + 3, 4096, 4096, 1, 32768, 1), # the shape of the recorded fault, in slabs
]


@pytest.mark.parametrize("rows,rowlen,N,nw,K,ew", SHAPES)
def test_every_offset_inside_its_buffer(lib, rows, rowlen, N, nw, K, ew):
    bad, partial_bytes, launches, rep = _walk(lib, rows, rowlen, N, nw, K, ew)
    assert bad == 0, rep
    assert partial_bytes <= 512 << 20


def test_shape_of_the_recorded_fault_in_its_original_single_launch(lib):
    rows = (1 << 20) + 3
    bad, partial_bytes, launches, rep = _walk(lib, rows, 4096, 4096, 1, 32768, 1, slab_segments=rows)
    assert launches == 1 and partial_bytes == rows * 64 * 256        # 17.18 GB of partial sums
    assert bad == 0, rep


def test_the_walk_notices_a_short_buffer(lib):
    """the same walk with a table one window short reports the gathers that leave it"""
    pb, nl = ctypes.c_size_t(0), ctypes.c_size_t(0)
    rep = ctypes.create_string_buffer(256)
    # claims 19 windows to the walk but sizes the table for N - 1 generators: every last column leaves it
    bad = lib.commit_geometry_check(64 * 128, 128, 127, 19, 8192, 8, 32768, 32, 24, ctypes.byref(pb), ctypes.byref(nl), rep, 256)
    assert bad > 0 and b"table word" in rep.value
