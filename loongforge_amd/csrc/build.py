"""Builds libdsa_hip.so (the C-ABI library of HIP kernels) for gfx950, in-tree.

    python -m loongforge_amd.csrc.build [--force]

hipcc cross-compiles without a GPU.  Objects and the shared library are written next to the
package (`loongforge_amd/libdsa_hip.so`) so that they travel with the source tree.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(PKG, "libdsa_hip.so")
OBJ_DIR = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wno-unused-result",
    # packed fp32 VALU ops are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _sources():
    return sorted(glob.glob(os.path.join(HERE, "*.hip")))


def _deps():
    return glob.glob(os.path.join(HERE, "*.h")) + glob.glob(os.path.join(os.path.dirname(PKG), "include", "*.h"))


def _compile(src, force):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    newest = max(os.path.getmtime(p) for p in [src] + _deps())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest:
        return obj, ""
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in (res.stdout + res.stderr).splitlines() if "not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    return obj, log


def build(force=False, verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = _sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(lambda s: _compile(s, force), srcs))
    objs = [o for o, _ in results]
    for _, log in results:
        if verbose and log.strip():
            print(log)
    newest = max(os.path.getmtime(o) for o in objs)
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < newest:
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("link failed:\n" + res.stdout + res.stderr)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
