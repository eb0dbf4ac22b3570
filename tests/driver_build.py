"""Builds the C++ drivers of the test-suite (tests/native/driver_flow.cpp, layer_flow.cpp, commit_flow.cpp,
programs_flow.cpp: programs in the reference's style against the host classes) with g++, for the curve GRAPE_CURVE names
(<name> for BLS12-381, <name>_bn254 for BN254)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
DRIVERS = ("driver_flow", "layer_flow", "commit_flow", "programs_flow")


def exe_path(curve, name="driver_flow"):
    return os.path.join(HERE, "native", name + ("_bn254" if curve == "bn254" else ""))


EXE = exe_path(os.environ.get("GRAPE_CURVE", "bls12_381"))


def build(curve=None, name="driver_flow"):
    curve = curve or os.environ.get("GRAPE_CURVE", "bls12_381")
    bn = curve == "bn254"
    suffix = "_bn254" if bn else ""
    exe = exe_path(curve, name)
    src = os.path.join(HERE, "native", name + ".cpp")
    host = os.path.join(ROOT, "grape_amd", "host")
    pkg = os.path.join(ROOT, "grape_amd")
    deps = [src, os.path.join(HERE, "native", "artefacts.hpp"), os.path.join(host, "libgrape_host%s.so" % suffix), os.path.join(pkg, "libgrape_hip%s.so" % suffix)]
    if os.path.exists(exe) and all(os.path.getmtime(d) <= os.path.getmtime(exe) for d in deps):
        return exe
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-Wno-unknown-pragmas", "-Wno-class-memaccess"]
                          + (["-DGRAPE_CURVE_BN254"] if bn else [])
                          + ["-o", exe, src, "-L" + host, "-lgrape_host" + suffix, "-L" + pkg, "-lgrape_hip" + suffix,
                             "-Wl,-rpath,$ORIGIN/../../grape_amd/host", "-Wl,-rpath,$ORIGIN/../../grape_amd"])
    return exe
