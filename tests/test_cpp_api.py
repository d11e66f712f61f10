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


# The reference's own example programs for this path, compiled unchanged against
# include/ and linked with the in-tree library (examples/example_utils.hpp:33-34
# includes "dnnl.hpp" and "dnnl_debug.h" from the top of the include directory).
# The sources stay where they are: the test only runs where the reference tree is
# mounted (the build container), and is skipped elsewhere.
REFERENCE_EXAMPLES = "/root/reference/examples"
EXAMPLES = ["tutorials/matmul/inference_int8_matmul.cpp", "tutorials/matmul/weights_decompression_matmul.cpp",
            "primitives/matmul.cpp", "matmul_perf.cpp"]


@pytest.mark.parametrize("rel", EXAMPLES)
def test_reference_example_compiles_and_links_unchanged(rel, tmp_path):
    src = os.path.join(REFERENCE_EXAMPLES, rel)
    if not os.path.exists(src):
        pytest.skip("reference examples are not mounted here")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "example.bin")
    cmd = ["g++", "-std=c++14", "-O0", "-I" + os.path.join(root, "include"), "-I" + REFERENCE_EXAMPLES, src, "-o", out,
           "-L" + os.path.join(root, "onednn_amd"), "-ldnnl_amd", "-Wl,-rpath," + os.path.join(root, "onednn_amd"),
           "-Wl,-rpath-link,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]


def test_debug_strings():
    import ctypes as C
    from onednn_amd import _capi
    L = _capi.lib()
    for fn in ("dnnl_status2str", "dnnl_dt2str", "dnnl_engine_kind2str", "dnnl_fmt_tag2str", "dnnl_alg_kind2str",
               "dnnl_prim_kind2str", "dnnl_fpmath_mode2str", "dnnl_scratchpad_mode2str", "dnnl_fmt_kind2str"):
        getattr(L, fn).restype = C.c_char_p
        getattr(L, fn).argtypes = [C.c_int]
    L.dnnl_runtime2str.restype = C.c_char_p
    # values of include/oneapi/dnnl/dnnl_common_types.h / dnnl_types.h
    assert L.dnnl_status2str(0) == b"success" and L.dnnl_status2str(3) == b"unimplemented"
    assert L.dnnl_dt2str(3) == b"f32" and L.dnnl_dt2str(10) == b"f8_e4m3" and L.dnnl_dt2str(12) == b"u4"
    assert L.dnnl_dt2str(0) == b"undef" and L.dnnl_dt2str(999) == b"unknown dt"
    assert L.dnnl_engine_kind2str(2) == b"gpu" and L.dnnl_engine_kind2str(0) == b"any"
    assert L.dnnl_fmt_tag2str(3) == b"ab" and L.dnnl_fmt_tag2str(15) == b"acb" and L.dnnl_fmt_tag2str(1) == b"any"
    assert L.dnnl_alg_kind2str(0x2c) == b"eltwise_swish" and L.dnnl_alg_kind2str(0x1fff0) == b"binary_add"
    assert L.dnnl_prim_kind2str(14) == b"matmul" and L.dnnl_prim_kind2str(1) == b"reorder"
    assert L.dnnl_fpmath_mode2str(1) == b"bf16" and L.dnnl_scratchpad_mode2str(1) == b"user"
    assert L.dnnl_fmt_kind2str(2) == b"blocked" and L.dnnl_runtime2str(1024) == b"HIP"
