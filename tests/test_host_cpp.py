"""The C++ host layer (pink::Trainer<...,true> / pink::Mapper<...,true> over the C ABI,
pink_amd/host/pink_hip_som.h) through its own test program tests/cpp/test_host.cpp."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_host")


def _bin():
    if not os.path.exists(BIN):
        from pink_amd import build
        build.build_host_test()
    return BIN


def test_argument_validation_needs_no_device():
    out = subprocess.run([_bin(), "args"], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr


@pytest.mark.gpu
def test_reference_known_answers_through_cpp_classes():
    out = subprocess.run([_bin(), "gpu"], capture_output=True, text=True, timeout=110)
    print(out.stdout, out.stderr, flush=True)
    assert out.returncode == 0, out.stdout + out.stderr
