"""Runs the C++ test driver of the host-side operator classes (tests/host/checker.cpp)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "host", "host_checker")


def _binary(allow_build):
    if not os.path.exists(BIN):
        if not allow_build:
            pytest.fail("tests/host/host_checker is not built (run __graft_entry__.build())")
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "megengine_amd", "host"), "-s"])
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "tests", "host"), "-s"])
    return BIN


def _run(mode, allow_build):
    r = subprocess.run([_binary(allow_build), mode], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout[-4000:]
    assert "ALL OK" in r.stdout


def test_host_classes_cpu():
    """layout deduction, validation errors and the algorithm surface; no device involved"""
    _run("--cpu", allow_build=True)


def test_abi_calls_from_many_threads():
    """tests/host/abi_stress.cpp: eight threads ask the host-side calls of the C ABI (deduce, query, usability, proofs) about
    1500 random descriptors, valid and invalid; every answer equals the one computed first.  The same driver runs under
    AddressSanitizer / UndefinedBehaviorSanitizer / ThreadSanitizer with `make -C tests/host sanitize` and `... tsan`."""
    _binary(allow_build=True)
    exe = os.path.join(ROOT, "tests", "host", "abi_stress")
    r = subprocess.run([exe, "8", "1500"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0 and "ALL OK" in r.stdout, r.stdout[-4000:]


@pytest.mark.gpu
def test_host_classes_gpu():
    """exec of every listed algorithm through the C++ classes, bit-exact against the CPU checker"""
    _run("--gpu", allow_build=False)
