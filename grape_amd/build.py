"""Builds the gfx950 shared libraries of the HIP kernels: grape_amd/libgrape_hip.so (BLS12-381,
the curve of the benchmark configurations) and grape_amd/libgrape_hip_bn254.so (BN254, the
reference's active curve; the same sources compiled with -DGRAPE_CURVE_BN254).

The library is built in-tree with hipcc (which cross-compiles without a GPU); nothing is
JIT-compiled at import time.  ``python -m grape_amd.build`` rebuilds it.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libgrape_hip.so")
SOURCES = ["runtime.hip", "fr_kernels.hip", "proto_kernels.hip", "round_kernels.hip", "g1_kernels.hip", "witness_kernels.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-std=c++17", "-O3", "--offload-arch=gfx950", "-fPIC",
         # packed-FP32 instruction forms are kept out of every device code object
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


# flavour -> (library, extra flags, object suffix)
FLAVOURS = {
    "bls12_381": (LIB, [], ".o"),
    "bn254": (os.path.join(HERE, "libgrape_hip_bn254.so"), ["-DGRAPE_CURVE_BN254"], ".bn254.o"),
}


def _compile(job):
    src, extra, suffix = job
    obj = os.path.join(CSRC, src.replace(".hip", suffix))
    cmd = [HIPCC] + FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj


def build(verbose=True, curves=("bls12_381", "bn254")):
    jobs = [(src,) + FLAVOURS[c][1:] for c in curves for src in SOURCES]
    with ThreadPoolExecutor(max_workers=8) as ex:
        objs = list(ex.map(_compile, jobs))
    for n, c in enumerate(curves):
        lib = FLAVOURS[c][0]
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", lib] + objs[n * len(SOURCES):(n + 1) * len(SOURCES)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("link failed:\n" + res.stderr)
        if verbose:
            print("built", lib)
    return LIB


if __name__ == "__main__":
    build(curves=tuple(sys.argv[1:]) or ("bls12_381", "bn254"))
    sys.exit(0)
