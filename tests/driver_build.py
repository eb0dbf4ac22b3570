"""Builds tests/native/driver_flow (a C++ driver in the reference's style) with g++, for the curve
GRAPE_CURVE names (driver_flow for BLS12-381, driver_flow_bn254 for BN254)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "native", "driver_flow.cpp")


def exe_path(curve):
    return os.path.join(HERE, "native", "driver_flow" + ("_bn254" if curve == "bn254" else ""))


EXE = exe_path(os.environ.get("GRAPE_CURVE", "bls12_381"))


def build(curve=None):
    curve = curve or os.environ.get("GRAPE_CURVE", "bls12_381")
    bn = curve == "bn254"
    suffix = "_bn254" if bn else ""
    exe = exe_path(curve)
    host = os.path.join(ROOT, "grape_amd", "host")
    pkg = os.path.join(ROOT, "grape_amd")
    deps = [SRC, os.path.join(host, "libgrape_host%s.so" % suffix), os.path.join(pkg, "libgrape_hip%s.so" % suffix)]
    if os.path.exists(exe) and all(os.path.getmtime(d) <= os.path.getmtime(exe) for d in deps):
        return exe
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-Wno-unknown-pragmas", "-Wno-class-memaccess"]
                          + (["-DGRAPE_CURVE_BN254"] if bn else [])
                          + ["-o", exe, SRC, "-L" + host, "-lgrape_host" + suffix, "-L" + pkg, "-lgrape_hip" + suffix,
                             "-Wl,-rpath,$ORIGIN/../../grape_amd/host", "-Wl,-rpath,$ORIGIN/../../grape_amd"])
    return exe
