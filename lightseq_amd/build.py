"""Builds ``liblightseq_hip.so`` (every HIP kernel + the C ABI) for gfx950 with hipcc.

``python -m lightseq_amd.build`` compiles each translation unit of ``csrc/`` to an
object file (in parallel) and links them into ``lightseq_amd/lib/``.  The GPU is not
needed: hipcc cross-compiles.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "_obj")
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "liblightseq_hip.so")

ARCH = "gfx950"
# -packed-fp32-ops off: hipcc must not form v_pk_{add,mul,fma}_f32 from float code.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=" + ARCH, "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def sources():
    out = []
    for root, _dirs, files in os.walk(CSRC):
        if os.path.basename(root) == "_obj":
            continue
        for f in sorted(files):
            if f.endswith(".hip") or f.endswith(".cpp"):
                out.append(os.path.join(root, f))
    return sorted(out)


def _compile_one(src):
    rel = os.path.relpath(src, CSRC).replace(os.sep, "_")
    obj = os.path.join(OBJ_DIR, os.path.splitext(rel)[0] + ".o")
    cmd = [_hipcc()] + HIPCC_FLAGS + ["-x", "hip", "-c", src, "-o", obj]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature; drop that one line
    log = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    return obj, log


def build_library(verbose=False, jobs=None):
    """Compile everything and link the shared library; returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(8, len(srcs))
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for obj, log in ex.map(_compile_one, srcs):
            objs.append(obj)
            if verbose and log.strip():
                print(log)
    cmd = [_hipcc(), "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o", LIB_PATH] + objs
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("link failed:\n" + p.stdout)
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(verbose=True)
    print("built", path)
    sys.exit(0)
