"""Builds the native code in-tree.

    python -m rwkv_lightning_cuda_amd.build [--force]

  csrc/*.hip -> librwkv_hip.so    gfx950 kernels behind the C ABI of include/rwkv_hip.h (hipcc; it
                                  cross-compiles without a GPU present).  No Python or torch dependency.
  host/*.cpp -> librwkv_host.so   the C++ host API of include/*.hpp (g++), linked against librwkv_hip.so.
  tests/cpp/*_test.cpp, *_bench.cpp -> tests/cpp/bin/*   test executables and measurement tools of the host API.
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
HOST_SRC = os.path.join(PKG_DIR, "host")
HOST_LIB_PATH = os.path.join(PKG_DIR, "librwkv_host.so")
TEST_SRC = os.path.join(REPO_DIR, "tests", "cpp")
TEST_BIN = os.path.join(TEST_SRC, "bin")
CXX = os.environ.get("CXX", "g++")
CXX_FLAGS = ["-std=c++17", "-O2", "-fPIC", "-Wall", "-I" + os.path.join(REPO_DIR, "include")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU ops are disabled for every device translation unit (see csrc/common.h users)
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# Kernels whose design depends on how many wavefronts fit a SIMD (mangled-name fragment -> required waves per SIMD):
# the compiler's resource report is checked at build time, so that a change that costs a few registers fails the
# build instead of silently halving the occupancy.  The one-row GEMV with the LayerNorm prologue needs two
# 1024-thread blocks per CU (all blocks of a launch resident at once), i.e. at most 64 registers.
# (template arguments: threads, prologue, format of the quantised problems 0 fp16 / 1 int8 / 2 int4, rows of x, row
# multiplier; two rows of int4 codes need more registers and run one block per CU; with the row multiplier 2 - int4
# launches with more blocks than CUs - a launch has one 1024-thread block per CU and needs 4 wavefronts per SIMD)
REQUIRED_OCCUPANCY = {"linear_gemv_row1_kernelILi1024ELb1ELi0ELi1ELi1E": 8, "linear_gemv_row1_kernelILi1024ELb1ELi1ELi1ELi1E": 8,
                      "linear_gemv_row1_kernelILi1024ELb1ELi2ELi1ELi1E": 8, "linear_gemv_row1_kernelILi1024ELb1ELi1ELi2ELi1E": 8,
                      "linear_gemv_row1_kernelILi1024ELb1ELi2ELi1ELi2E": 4, "linear_gemv_row1_kernelILi1024ELb1ELi2ELi2ELi2E": 4}


def _check_occupancy(src, stderr_text):
    name = None
    for line in stderr_text.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif "Occupancy [waves/SIMD]:" in line and name:
            got = int(line.split("Occupancy [waves/SIMD]:")[1].split()[0])
            for frag, need in REQUIRED_OCCUPANCY.items():
                if frag in name and got < need:
                    raise RuntimeError("%s: kernel %s fits %d wavefronts per SIMD, its design needs %d "
                                       "(register count went up)" % (src, name, got, need))


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
    cmd = [HIPCC] + HIP_FLAGS + ["-Rpass-analysis=kernel-resource-usage", "-c", spath, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in proc.stderr.splitlines()
                    if "packed-fp32-ops" not in l and "kernel-resource-usage" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    _check_occupancy(src, proc.stderr)
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


def _run(cmd, what):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("%s failed:\n%s" % (what, proc.stderr))


def build_host(verbose=True):
    """Compiles host/*.cpp into librwkv_host.so (needs librwkv_hip.so to be built).  Returns its path."""
    srcs = sorted(os.path.join(HOST_SRC, f) for f in os.listdir(HOST_SRC) if f.endswith(".cpp"))
    cmd = ([CXX] + CXX_FLAGS + ["-shared", "-o", HOST_LIB_PATH] + srcs
           + ["-L" + PKG_DIR, "-lrwkv_hip", "-ldl", "-pthread", "-Wl,-rpath,$ORIGIN"])
    _run(cmd, "host library build")
    if verbose:
        print("built", HOST_LIB_PATH)
    return HOST_LIB_PATH


def host_test_names():
    return sorted(f[:-4] for f in os.listdir(TEST_SRC) if f.endswith("_test.cpp"))


def host_tool_names():
    """Measurement tools over the host API (run by bench.py), built like the tests."""
    return sorted(f[:-4] for f in os.listdir(TEST_SRC) if f.endswith("_bench.cpp"))


def build_host_tests(verbose=True):
    """Compiles every tests/cpp/*_test.cpp into tests/cpp/bin/ (needs both libraries)."""
    os.makedirs(TEST_BIN, exist_ok=True)
    rpath = "-Wl,-rpath," + PKG_DIR + ":$ORIGIN/../../../rwkv_lightning_cuda_amd"
    outs = []
    for name in host_test_names() + host_tool_names():
        out = os.path.join(TEST_BIN, name)
        cmd = ([CXX] + CXX_FLAGS + ["-I" + TEST_SRC, os.path.join(TEST_SRC, name + ".cpp"), "-o", out,
                                   "-L" + PKG_DIR, "-lrwkv_host", "-lrwkv_hip", "-pthread", rpath])
        _run(cmd, "test build " + name)
        outs.append(out)
    if verbose:
        print("built", len(outs), "host test executables")
    return outs


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
    build_host()
    build_host_tests()
