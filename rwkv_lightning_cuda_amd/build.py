"""Builds the gfx950 kernel library (csrc/*.hip -> librwkv_hip.so) in-tree with hipcc.

    python -m rwkv_lightning_cuda_amd.build [--force]

hipcc cross-compiles for gfx950 without a GPU present.  The shared library has no Python or torch
dependency: it exports only the C ABI declared in include/rwkv_hip.h.
"""
import concurrent.futures
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(PKG_DIR, "build")
LIB_PATH = os.path.join(PKG_DIR, "librwkv_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU ops are disabled for every device translation unit (see csrc/common.h users)
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers_mtime():
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    paths.append(os.path.join(REPO_DIR, "include", "rwkv_hip.h"))
    return max(os.path.getmtime(p) for p in paths)


def _compile(src, force):
    obj = os.path.join(OBJ_DIR, src[:-4] + ".o")
    spath = os.path.join(CSRC, src)
    if (not force and os.path.exists(obj)
            and os.path.getmtime(obj) > max(os.path.getmtime(spath), _headers_mtime())):
        return obj, ""
    cmd = [HIPCC] + HIP_FLAGS + ["-c", spath, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    return obj, log


def build_all(force=False, verbose=True):
    """Compiles every .hip file (in parallel) and links librwkv_hip.so.  Returns the library path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        results = list(pool.map(lambda s: _compile(s, force), srcs))
    objs = [r[0] for r in results]
    for src, (_, log) in zip(srcs, results):
        if log.strip() and verbose:
            print("[%s]\n%s" % (src, log), file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stderr)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
