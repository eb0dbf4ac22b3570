"""Builds the C++ host libraries with g++ and links each against the HIP kernel library of its
curve: grape_amd/host/libgrape_host.so (BLS12-381) and libgrape_host_bn254.so (BN254, the same
sources with -DGRAPE_CURVE_BN254).  Host code contains no HIP calls: it reaches the GPU only through the
C ABI of include/grape_hip.h."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libgrape_host.so")
SOURCES = ["fr.cpp", "polynomial.cpp", "fr_tensor.cpp", "ec_operation.cpp", "hyrax.cpp", "prove.cpp", "tlookup.cpp", "ioutils.cpp", "timer.cpp", "witness.cpp", "host_capi.cpp"]


# flavour -> (library, extra compiler flags, kernel library to link)
FLAVOURS = {
    "bls12_381": (LIB, [], "grape_hip"),
    "bn254": (os.path.join(HERE, "libgrape_host_bn254.so"), ["-DGRAPE_CURVE_BN254"], "grape_hip_bn254"),
}


def build(verbose=True, curves=("bls12_381", "bn254")):
    for c in curves:
        lib, extra, kernels = FLAVOURS[c]
        cmd = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wno-unused-function", "-Wno-unknown-pragmas", "-Wno-class-memaccess"] + extra + \
              ["-o", lib] + [os.path.join(HERE, s) for s in SOURCES] + \
              ["-L" + PKG, "-l" + kernels, "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + PKG]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("g++ failed:\n" + res.stderr)
        if verbose:
            if res.stderr.strip():
                print(res.stderr)
            print("built", lib)
    return LIB


if __name__ == "__main__":
    build(curves=tuple(sys.argv[1:]) or ("bls12_381", "bn254"))
    sys.exit(0)
