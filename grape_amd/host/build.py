"""Builds the C++ host library (grape_amd/host/libgrape_host.so) with g++ and links it against
the HIP kernel library.  Host code contains no HIP calls: it reaches the GPU only through the
C ABI of include/grape_hip.h."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libgrape_host.so")
SOURCES = ["fr.cpp", "polynomial.cpp", "fr_tensor.cpp", "ec_operation.cpp", "hyrax.cpp", "prove.cpp", "tlookup.cpp", "ioutils.cpp", "timer.cpp", "host_capi.cpp"]


def build(verbose=True):
    cmd = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wno-unused-function", "-Wno-unknown-pragmas", "-Wno-class-memaccess",
           "-o", LIB] + [os.path.join(HERE, s) for s in SOURCES] + \
          ["-L" + PKG, "-lgrape_hip", "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + PKG]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("g++ failed:\n" + res.stderr)
    if verbose:
        if res.stderr.strip():
            print(res.stderr)
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
