"""Build recipe of libspgt_hip.so (hipcc, gfx950 only).

`python -m spgt_amd.build` compiles every source under csrc/ into
spgt_amd/libspgt_hip.so.  hipcc cross-compiles, so no GPU is needed.
"""
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libspgt_hip.so")

SOURCES = [
    "spgt_host.cpp",
    "attn_fused.hip",
    "attn_fm.hip",
    "attn_backward.hip",
    "splitk_gemm.hip",
    "projection.hip",
    "datamove.hip",
    "spectral.hip", "spectral_dft.hip", "linear.hip",
]

# Packed fp32 VALU forms (v_pk_*_f32) are switched off for all device code.
HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def build(verbose: bool = False) -> str:
    """Compile the library from scratch and return its path."""
    srcs = [os.path.join(CSRC_DIR, s) for s in SOURCES]
    tmp = LIB_PATH + ".tmp"
    cmd = [find_hipcc(), *HIPCC_FLAGS, "-x", "hip", *srcs, "-o", tmp]
    proc = subprocess.run(cmd, cwd=CSRC_DIR, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the device-only feature name and says so.
    log = "\n".join(l for l in proc.stdout.splitlines() if "not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + log)
    if verbose and log.strip():
        print(log)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
