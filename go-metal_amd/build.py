"""Builds libgometal_hip.so (HIP kernels + C ABI + host-side optimizer mirror) for gfx950.

hipcc cross-compiles without a GPU, so this runs in any container with ROCm.
"""
import glob
import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libgometal_hip.so")

# -ffp-contract=off: every written fp32 operation rounds once (no FMA fusion), which is what
#   makes the kernels bit-identical to the reference equations; it also covers the host code
#   that computes the step scalars.
# -fhip-fp32-correctly-rounded-divide-sqrt: IEEE division and square root on the device
#   (hipcc's default, stated explicitly because the parity bar depends on it).
# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 instructions.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def sources():
    srcs = sorted(glob.glob(os.path.join(PKG_DIR, "csrc", "*.hip")))
    srcs += sorted(glob.glob(os.path.join(PKG_DIR, "csrc", "*.cpp")))
    srcs += sorted(glob.glob(os.path.join(PKG_DIR, "host", "*.cpp")))
    return srcs


def build(verbose=True):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc] + HIPCC_FLAGS + ["-x", "hip"] + sources() + ["-o", LIB_PATH, "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


if __name__ == "__main__":
    build()
