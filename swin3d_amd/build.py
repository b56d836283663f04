"""Builds swin3d_amd/libswin3d_amd.so with hipcc for gfx950.

Usage: python -m swin3d_amd.build [--force]
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libswin3d_amd.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = ["api_common.hip", "attn_fwd.hip", "attn_sweep.hip", "attn_bwd.hip",
           "window_index.hip", "knn.hip", "layernorm.hip"]

# packed-fp32 VALU forms are disabled for every device compilation unit
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-munsafe-fp-atomics",   # LDS float adds as one ds_add_f32 instead of a compare-and-swap loop
    "-Wno-unused-command-line-argument",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    extra = os.environ.get("S3D_HIPCC_EXTRA", "").split()   # e.g. -D switches of a kernel experiment
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass reports that it does not know the device-only target feature
    log = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{log}")
    return obj, log


def build(force=True, verbose=False):
    """Compile every HIP source and link the shared library (always recompiles when force)."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    if not force and os.path.exists(LIB):
        newest = max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC))
        if os.path.getmtime(LIB) >= newest:
            return LIB
    with ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(_compile, SOURCES))
    for _, log in results:
        if verbose and log.strip():
            print(log)
    objs = [o for o, _ in results]
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}")
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or True, verbose=True))
