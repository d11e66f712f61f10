"""Builds tests/cpp/dnnl_hpp_check.cpp against the in-tree library: the C++
header layer is header-only, so this is also its compile check."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SRC = os.path.join(HERE, "dnnl_hpp_check.cpp")
BIN = os.path.join(HERE, "dnnl_hpp_check.bin")


def build():
    cmd = ["g++", "-std=c++14", "-O1", "-Wall", "-I" + os.path.join(ROOT, "include"), SRC, "-o", BIN,
           "-L" + os.path.join(ROOT, "onednn_amd"), "-ldnnl_amd",
           "-Wl,-rpath,$ORIGIN/../../onednn_amd", "-Wl,-rpath-link,/opt/rocm/lib"]
    subprocess.run(cmd, check=True)
    return BIN


def binary():
    """The built checker; compiled only when it is not there yet."""
    return BIN if os.path.exists(BIN) else build()
