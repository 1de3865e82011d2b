"""Compile the HIP sources under ``falkon_amd/csrc`` into ``falkon_amd/lib/libfalkon_amd.so``.

The library is built for gfx950 only, with plain ``hipcc`` (no torch headers: the
C ABI takes raw pointers), one object per source (and kernel function) compiled in parallel.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libfalkon_amd.so")
OBJ_DIR = os.path.join(_HERE, "build")

# The sources that evaluate the kernel function are compiled once per function: -DFLK_KF=0..4
# (Gaussian, Laplacian, Matern 3/2, Matern 5/2, the Laplacian's derivative weight).
KERNEL_FNS = (0, 1, 2, 3, 4)
PER_KERNEL_FN = ["mmv_small_f32.hip", "mmv_small_f32_fold.hip", "mmv_small_f32_wide.hip", "mmv_small_f64.hip", "mmv_small_f64_wide.hip", "mmv_large.hip", "fmm.hip",
                 "mmv_split.hip", "mmv_split_wide.hip", "mmv_split_large.hip"]
# Longest compiles first (the many-column fp32 kernel takes as long as all the other sources of its kernel function
# together), so that the parallel build does not end on one of them running alone.
SOURCES = [(src, kf) for src in PER_KERNEL_FN for kf in KERNEL_FNS]
SOURCES.sort(key=lambda job: {"mmv_small_f32_wide.hip": 0, "mmv_small_f32.hip": 1, "mmv_small_f32_fold.hip": 2}.get(job[0], 3))
SOURCES += [("api.hip", None), ("pack.hip", None), ("pack_split.hip", None), ("cg.hip", None), ("trsv.hip", None), ("potrf.hip", None)]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # keep MFMA accumulators in VGPRs: the epilogue reads every accumulator with VALU ops
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the falkon_amd native library needs ROCm's hipcc to build")


def _headers_mtime() -> float:
    hdrs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".h", ".inc"))]
    hdrs.append(os.path.join(_HERE, "..", "include", "falkon_amd.h"))
    return max(os.path.getmtime(h) for h in hdrs)


def _compile(job) -> str:
    src, kf, only_changed = job
    stem = os.path.splitext(src)[0] + ("" if kf is None else f"_kf{kf}")
    obj = os.path.join(OBJ_DIR, stem + ".o")
    if only_changed and os.path.exists(obj):
        if os.path.getmtime(obj) > max(os.path.getmtime(os.path.join(CSRC, src)), _headers_mtime()):
            return obj
    defines = [] if kf is None else [f"-DFLK_KF={kf}"]
    cmd = [_hipcc(), *HIPCC_FLAGS, *defines, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src} {' '.join(defines)}:\n{res.stderr}")
    return obj


def build(verbose: bool = True, jobs: int = 0, only_changed: bool = False) -> str:
    """Compile every source (always, also when a library is already there) and link.  With ``only_changed`` an
    object newer than its source and every header is kept (a developer's shortcut; the default rebuilds all)."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, [(src, kf, only_changed) for src, kf in SOURCES]))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[falkon_amd] built {LIB_PATH}", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build(only_changed="--changed" in sys.argv)
