"""Compile the HIP library for gfx950 (cross-compiles without a GPU).

    python -m pink_amd.build

writes pink_amd/lib/libpink_hip.so.  The flags matter for parity with the CPU path:
no floating-point contraction (products and sums of the rotation and update kernels
round separately; the distance kernel asks for its fused multiply-add explicitly) and
no packed-FP32 instructions.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SOURCES = [os.path.join(HERE, "csrc", "pink_hip.hip"), os.path.join(HERE, "csrc", "update_factors.cpp")]
# Compiled on its own with the MFMA accumulators in the architectural vector registers: its
# distance kernel fills all 256 accumulation registers with resident SOM fragments (which the MFMA
# reads as operands) and post-processes the accumulators on the vector ALU, which cannot read
# accumulation registers.  The other MFMA kernels want the default (accumulators there).
SYM_SOURCE = os.path.join(HERE, "csrc", "mfma_u8_sym.hip")
SYM_FLAGS = ["-mllvm", "-amdgpu-mfma-vgpr-form"]
OUT = os.path.join(HERE, "lib", "libpink_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    "-I" + os.path.join(ROOT, "include"),
]


def build(verbose=False, extra=()):
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    obj_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    objects, cmds = [], []
    for src in SOURCES + [SYM_SOURCE]:
        obj = os.path.join(HERE, "lib", os.path.splitext(os.path.basename(src))[0] + ".o")
        flags = obj_flags + (SYM_FLAGS if src == SYM_SOURCE else [])
        cmds.append([hipcc] + flags + list(extra) + ["-c", src, "-o", obj])
        objects.append(obj)
    cmds.append([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objects + ["-o", OUT])
    for cmd in cmds:
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return OUT


HOST_TEST_SRC = os.path.join(ROOT, "tests", "cpp", "test_host.cpp")
HOST_TEST_BIN = os.path.join(ROOT, "tests", "cpp", "test_host")


def build_host_test(verbose=False):
    """Compile the C++ Trainer/Mapper mirror (pink_amd/host) and its test with the host compiler."""
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-Wall", "-Wextra",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "host"),
           HOST_TEST_SRC, "-o", HOST_TEST_BIN, "-L" + os.path.join(HERE, "lib"), "-lpink_hip",
           "-Wl,-rpath,$ORIGIN/../../pink_amd/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return HOST_TEST_BIN


if __name__ == "__main__":
    build(verbose=True, extra=sys.argv[1:])
    build_host_test(verbose=True)
