"""Builds the shared library of the MI355X quantized-matmul path.

hipcc cross-compiles every translation unit for gfx950 (no GPU needed) and
links one in-tree shared object, onednn_amd/libdnnl_amd.so, which exports the
dnnl_* C API subset and the qmm_* kernel-level C ABI.

Flags of note:
  -ffp-contract=off   the epilogue must round every float step separately;
  -Xclang -target-feature -Xclang -packed-fp32-ops
                      keeps the compiler from forming packed FP32 instructions.
"""
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libdnnl_amd.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wno-inline-asm",
          "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
          "-Wall", "-Wno-unused-function", "-Wno-pass-failed"]
DEVICE = ["--offload-arch=gfx950", "-ffp-contract=off",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# (source, object suffix, extra defines)
# the decode kernel takes its address-forming arguments preloaded into scalar
# registers at wave launch (leading kernel arguments, at most 14 dwords)
PRELOAD = ["-mllvm", "-amdgpu-kernarg-preload-count=14"]
UNITS = [("qmm_generic.hip", "", []), ("qmm_gemv_w4.hip", "", PRELOAD),
         ("qmm_pack.hip", "", []), ("qmm_quantize.hip", "", []),
         ("qmm_dispatch.hip", "", []), ("qmm_measure.hip", "", PRELOAD), ("qmm_softmax.hip", "", []), ("qmm_sdpa.hip", "", []),
         ("qmm_gemm_b8.hip", "", []),
         ("qmm_gemm_b8x.hip", "", []), ("qmm_gemm_w4a8.hip", "", []), ("qmm_gemv_b8.hip", "", []), ("qmm_gemm_w4f.hip", "", []), ("qmm_gemm_f16.hip", "", []),
         ("dnnl_core.cpp", "", []), ("dnnl_primitives.cpp", "", [])]
# the tiled GEMM is instantiated once per tile configuration, each in its own
# object so the instantiations compile in parallel
GEMM_VARIANTS = [1, 2, 3]
for v in GEMM_VARIANTS:
    for k in (0, 1, 2):
        UNITS.append(("qmm_gemm_b8.hip", "_v%d_k%d" % (v, k),
                      ["-DQMM_GEMM_VARIANT=%d" % v, "-DQMM_GEMM_KIND=%d" % k]))
# likewise the 256 x 256 kernels: int8, short-K int8, fp8, int8 on 16 x 16 MFMAs
# (even and odd numbers of k-steps), fp8 on 16 x 16 MFMAs, int8 with two workgroups per CU
for v in (1, 2, 3, 4, 5, 6, 7):
    UNITS.append(("qmm_gemm_b8x.hip", "_p%d" % v, ["-DQMM_B8X_PART=%d" % v]))
for v in (1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14):
    UNITS.append(("qmm_gemm_w4a8.hip", "_p%d" % v, ["-DQMM_W4A8_PART=%d" % v]))
# f16 x 8-bit weights on the 256 x 256 design: even and odd numbers of k-steps
for v in (0, 1):
    UNITS.append(("qmm_gemm_f16w8.hip", "_p%d" % v, ["-DQMM_F16W8_PART=%d" % v]))
# the tiled decompression kernel per activation type and weights width
for v in (0, 1, 2, 3):
    UNITS.append(("qmm_gemm_w4f.hip", "_p%d" % v, ["-DQMM_W4F_PART=%d" % v]))
# longest first, so that the pool finishes together
UNITS.sort(key=lambda u: 0 if "w4a8" in u[0] or ("w4f" in u[0] and u[1]) else (1 if u[1] else 2))


def _compile(unit):
    src, suffix, defs = unit
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + suffix + ".o")
    cmd = [HIPCC] + COMMON + defs
    if src.endswith(".hip"):
        cmd += DEVICE
    else:
        cmd += ["-x", "hip", "--offload-host-only"] if False else []
    cmd += ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True)
    out = "\n".join(l for l in r.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "warning generated" not in l)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s" % (" ".join(cmd), out))
    return obj, out


def build(verbose=False, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 4)
    objs = []
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        for obj, out in ex.map(_compile, UNITS):
            objs.append(obj)
            if verbose and out.strip():
                print(out)
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
