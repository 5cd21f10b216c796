"""The C++ host mirror (include/rustorch_attn.hpp) through its own test program (tests/cpp): error enums and
their order on the CPU, small forwards against a double-precision loop on the GPU."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CPP = os.path.join(HERE, "cpp")


def _binary():
    subprocess.check_call(["make", "-s", "-C", CPP, "host_mirror_test"])
    return os.path.join(CPP, "host_mirror_test")


def test_cpp_error_surface_needs_no_gpu():
    r = subprocess.run([_binary(), "errors"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.strip().endswith("ok")


@pytest.mark.gpu
def test_cpp_forward_matches_double_precision_loop():
    r = subprocess.run([_binary(), "gpu"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.strip().endswith("ok")
