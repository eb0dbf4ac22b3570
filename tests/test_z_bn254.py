"""The BN254 instantiation (the reference's active curve, include/field/alt_bn128.cuh,
include/ec_operation.cuh:3-6): the same test-suite run once more in a child process with
GRAPE_CURVE=bn254, which switches the big-integer references, the CPU oracle, the known-answer
vectors and the loaded libraries (libgrape_hip_bn254.so / libgrape_host_bn254.so) to that curve.
One curve per process: the libraries fix it at compile time."""
import os
import subprocess
import sys
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
pytestmark = pytest.mark.skipif(os.environ.get("GRAPE_CURVE", "bls12_381") != "bls12_381",
                                reason="already running under a non-default curve")


def _run(marker, timeout):
    env = dict(os.environ, GRAPE_CURVE="bn254")
    cmd = [sys.executable, "-u", "-m", "pytest", HERE, "-q", "-x", "-m", marker, "--timeout", "120",
           "--timeout-method", "thread", "-p", "no:cacheprovider", "--deselect", os.path.join(HERE, "test_z_bn254.py")]
    res = subprocess.run(cmd, env=env, capture_output=True, text=True, timeout=timeout)
    tail = "\n".join(res.stdout.splitlines()[-25:]) + "\n" + "\n".join(res.stderr.splitlines()[-10:])
    assert res.returncode == 0, tail
    assert " passed" in res.stdout and "failed" not in res.stdout.splitlines()[-1], tail


def test_cpu_suite_under_bn254():
    """oracle vs big integers and the BN254 known-answer vectors, the 28-/26-bit limb arithmetic on
    the host, the exported symbols of the BN254 libraries"""
    _run("not gpu", 900)


@pytest.mark.gpu
def test_gpu_suite_under_bn254():
    """every GPU parity test (field, curve, commitments, fold, sumcheck, logUp, host classes)
    against the BN254 oracle, bit-exact, through the C ABI of libgrape_hip_bn254.so"""
    _run("gpu", 900)
