"""Builds libmyea_hip.so (gfx950) in-tree with hipcc.  `python -m myea_amd.build` or build()."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(CSRC, "libmyea_hip.so")
HIP_SOURCES = ["myea_gemm.hip", "myea_elementwise.hip", "myea_lstm.hip", "myea_lstm_fused.hip", "myea_lstm_resident.hip", "myea_ceilings.hip", "myea_net.hip"]
C_SOURCES = ["myea_layout.c"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed-FP32 instructions are switched off for every device TU
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + "\n")
        raise RuntimeError("build step failed: " + " ".join(cmd[:2]))
    return proc.stdout


def build(verbose=False):
    """Compile every HIP source for gfx950 and link the shared library (always rebuilds)."""
    from concurrent.futures import ThreadPoolExecutor

    def compile_hip(src):
        obj = os.path.join(CSRC, src + ".o")
        out = _run([HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=4) as pool:
        objs = list(pool.map(compile_hip, HIP_SOURCES))
    for src in C_SOURCES:
        obj = os.path.join(CSRC, src + ".o")
        _run(["gcc", "-O2", "-fPIC", "-std=c11", "-Wall", "-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    # the C++ adaptor's check programs (host code only; link the C ABI)
    root = os.path.dirname(HERE)
    for name in ("adaptor_check", "dataset_check", "checkpoint_check"):
        _run(["g++", "-O2", "-std=c++17", "-Wall", "-fopenmp", os.path.join(root, "tests", "cpp", name + ".cpp"), "-o",
              os.path.join(root, "tests", "cpp", name), "-L" + CSRC, "-lmyea_hip", "-Wl,-rpath," + CSRC,
              "-Wl,-rpath,$ORIGIN/../../myea_amd/csrc"])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
