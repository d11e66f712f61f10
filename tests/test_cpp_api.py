"""The C++ header layer (include/oneapi/dnnl/dnnl.hpp) driven from a C++
program, as an application of the reference's C++ API would use it."""
import os
import subprocess
import sys

import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp"))
import build_check  # noqa: E402


def _run(mode, env_extra=None):
    env = dict(os.environ)
    env.update(env_extra or {})
    r = subprocess.run([build_check.binary(), mode], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stdout + r.stderr
    return r.stdout


def test_cpp_header_descriptors_and_attributes():
    out = _run("host", {"DNNL_AMD_DESCRIPTOR_ONLY": "1"})
    assert "host ok" in out


@pytest.mark.gpu
def test_cpp_header_matmul_and_inner_product():
    out = _run("gpu")
    assert "gpu ok" in out
    assert "hip:gfx950" in out
