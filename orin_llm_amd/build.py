"""Builds liborin_fa.so (HIP kernels + C ABI + llm::cuda shim) for gfx950, in-tree."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liborin_fa.so")
SOURCES = [os.path.join(HERE, "csrc", "fa_kernels.hip"), os.path.join(HERE, "csrc", "llm_cuda_shim.cpp")]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-exceptions",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose=False):
    cmd = [HIPCC] + FLAGS + SOURCES + ["-o", LIB]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
    if verbose:
        print(" ".join(cmd))
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
