"""Build libxnor_nn.so (HIP, gfx950 only) in-tree: ``python -m xnor_nn_amd.build``.

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
"""
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "lib", "libxnor_nn.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # every product and sum of the float reductions is rounded on its own, like the CPU
    # library this replaces
    "-ffp-contract=off",
    "-fno-fast-math",
    # do not let the compiler form packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libxnor_nn.so needs the ROCm toolchain")
    return exe


def build(verbose=True, extra=(), out=OUT):
    sources = sorted(glob.glob(os.path.join(SRC, "*.hip")))
    os.makedirs(os.path.dirname(out), exist_ok=True)
    cmd = [hipcc()] + FLAGS + list(extra) + [
        "-I" + os.path.join(ROOT, "include"), "-I" + SRC] + sources + ["-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


if __name__ == "__main__":
    build(extra=sys.argv[1:])
