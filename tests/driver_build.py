"""Builds tests/native/driver_flow (a C++ driver in the reference's style) with g++."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "native", "driver_flow.cpp")
EXE = os.path.join(HERE, "native", "driver_flow")


def build():
    host = os.path.join(ROOT, "grape_amd", "host")
    pkg = os.path.join(ROOT, "grape_amd")
    deps = [SRC, os.path.join(host, "libgrape_host.so"), os.path.join(pkg, "libgrape_hip.so")]
    if os.path.exists(EXE) and all(os.path.getmtime(d) <= os.path.getmtime(EXE) for d in deps):
        return EXE
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-Wno-unknown-pragmas", "-Wno-class-memaccess", "-o", EXE, SRC,
                           "-L" + host, "-lgrape_host", "-L" + pkg, "-lgrape_hip",
                           "-Wl,-rpath,$ORIGIN/../../grape_amd/host", "-Wl,-rpath,$ORIGIN/../../grape_amd"])
    return EXE
