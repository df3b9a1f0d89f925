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
# The same library with the hand-written MFMA statements of linear.hip replaced by the compiler's intrinsic:
# test infrastructure (tests compare the two bit for bit), never loaded by the package.
CHECK_LIB_PATH = os.path.join(PKG_DIR, "libspgt_hip_mfma_check.so")
CHECK_SOURCE, CHECK_DEFINE = "linear.hip", "-DSPGT_MFMA_BUILTIN=1"

SOURCES = [
    "spgt_host.cpp",
    "attn_fused.hip",
    "attn_fused_backward.hip",
    "attn_fm.hip",
    "attn_backward.hip",
    "splitk_gemm.hip",
    "projection.hip",
    "datamove.hip",
    "spectral.hip", "spectral_dft.hip", "linear.hip", "linear_backward.hip",
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


def _newest_header_mtime() -> float:
    hdrs = [os.path.join(CSRC_DIR, f) for f in os.listdir(CSRC_DIR) if f.endswith(".h")]
    hdrs.append(os.path.join(PKG_DIR, "..", "include", "spgt_hip.h"))
    return max(os.path.getmtime(h) for h in hdrs)


def build(verbose: bool = False, incremental: bool = False, jobs: int = 8) -> str:
    """Compile the library and return its path.  Every source is compiled to an object of its own
    (up to `jobs` at a time) and the objects are linked.  By default everything is recompiled;
    with `incremental` an object newer than its source and every header is kept."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = find_hipcc()
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    hdr_mtime = _newest_header_mtime()
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]

    def clean(text):
        # hipcc's host pass does not know the device-only feature name and says so.
        return "\n".join(l for l in text.splitlines() if "not a recognized feature" not in l)

    def compile_one(job):
        name, defines, suffix = job
        src = os.path.join(CSRC_DIR, name)
        obj = os.path.join(obj_dir, name + suffix + ".o")
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), hdr_mtime):
            return obj, ""
        cmd = [hipcc, *flags, *defines, "-x", "hip", "-c", src, "-o", obj]
        proc = subprocess.run(cmd, cwd=CSRC_DIR, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + clean(proc.stdout))
        return obj, clean(proc.stdout)

    work = [(name, [], "") for name in SOURCES] + [(CHECK_SOURCE, [CHECK_DEFINE], ".builtin")]
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        results = list(pool.map(compile_one, work))
    objs = [o for o, _ in results[:-1]]
    check_objs = [results[-1][0] if name == CHECK_SOURCE else o for name, o in zip(SOURCES, objs)]
    log = "\n".join(t for _, t in results if t.strip())
    for path, members in ((LIB_PATH, objs), (CHECK_LIB_PATH, check_objs)):
        tmp = path + ".tmp"
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *members, "-o", tmp]
        proc = subprocess.run(cmd, cwd=CSRC_DIR, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError("link failed:\n" + " ".join(cmd) + "\n" + clean(proc.stdout))
        os.replace(tmp, path)
    if verbose and log.strip():
        print(log)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True, incremental="--incremental" in sys.argv))
    sys.exit(0)
