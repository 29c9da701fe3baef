"""Compile the gfx950 kernels into ``blockgtq_amd/_lib/libbgtq.so`` with hipcc.

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain
is installed.  The library is kept in-tree next to the package.
"""
import os
import shutil
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_DIR = os.path.join(_HERE, "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libbgtq.so")

ARCH = "gfx950"
COMMON = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-fhip-fp32-correctly-rounded-divide-sqrt"]
# source file -> extra flags.  The encoders promise a fixed floating-point
# evaluation order, so nothing in that file may be contracted into an fma
# behind the author's back.
SOURCES = {
    "bgtq_encode.hip": ["-ffp-contract=off"],
    "bgtq_decode.hip": ["-fno-strict-aliasing"],
    # LDS tiles are written as 128-bit / 16-bit words and read back as 32-bit words
    "bgtq_decode_seg.hip": ["-fno-strict-aliasing"],
    "bgtq_dequant.hip": [],
    "bgtq_prefill.hip": ["-fno-strict-aliasing"],
}


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the kernels need the ROCm toolchain")
    return exe


def build(verbose=False):
    """Compile every HIP source and link the shared library.  Returns its path."""
    hipcc = _hipcc()
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    for src, extra in SOURCES.items():
        obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
        cmd = [hipcc] + COMMON + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{res.stderr}")
        objs.append(obj)
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC"] + objs + ["-o", tmp]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
