"""Runs the C++ operator-API test program (tests/cpp/test_device_api.cpp): the
reference's testbed sweep, its three examples and its known-answer vector,
through cuasr::gemm::device::Srgemm / SrgemmSplitKParallel."""
import os
import subprocess

import pytest

import build_cpp

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_operator_api(lib):
    r = subprocess.run([build_cpp.ensure("test_device_api")], capture_output=True, text=True, timeout=600)
    print(r.stdout[-4000:])
    print(r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-4000:]
    assert "0 failed" in r.stdout


def test_cpp_user_defined_functors(lib):
    """tests/cpp/test_user_functor.hip: device::Srgemm with functors the library has no operator for (the
    kernel is built from the functors, in a translation unit compiled by hipcc) against the host reference."""
    r = subprocess.run([build_cpp.ensure("test_user_functor")], capture_output=True, text=True, timeout=600)
    print(r.stdout[-4000:])
    print(r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-4000:]
    assert "0 failed" in r.stdout


def test_cpp_reference_call_sites(lib):
    """tests/cpp/test_reference_call_sites.hip: the three call shapes of the reference's examples, spelled with
    cutlass:: names, a user functor with Array overloads and a cutlass::device_memory workspace."""
    r = subprocess.run([build_cpp.ensure("test_reference_call_sites")], capture_output=True, text=True, timeout=600)
    print(r.stdout[-4000:])
    print(r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-4000:]
    assert "0 failed" in r.stdout
