"""Build step of the HIP library: one hipcc line, output kept in-tree under lib/."""
import os
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
SOURCE = os.path.join(_PKG, "csrc", "cachegen_hip.hip")
LIBRARY = os.path.join(_PKG, "lib", "libcachegen_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",                     # float32 steps are rounded one by one
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(_ROOT, "include"),
]


def build_library(verbose=False):
    """Compile csrc/cachegen_hip.hip for gfx950 into lib/libcachegen_hip.so."""
    os.makedirs(os.path.dirname(LIBRARY), exist_ok=True)
    hipcc = os.environ.get("HIPCC", "hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", LIBRARY, SOURCE]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout)
    if verbose:
        print(res.stdout)
    return LIBRARY


if __name__ == "__main__":
    print(build_library(verbose=True))
