"""Builds the HIP libraries for gfx950, in-tree.

    python -m loongforge_amd.csrc.build [--force]

libdsa_hip.so    the C-ABI library of kernels (include/dsa_hip.h): every csrc/*.hip
libdsa_bench.so  measurement aids that only the benchmark loads (include/dsa_hip_bench.h):
                 csrc/bench/*.hip plus the error-state object

hipcc cross-compiles without a GPU.  Objects and the shared libraries are written next to the
package (`loongforge_amd/*.so`) so that they travel with the source tree.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(PKG, "libdsa_hip.so")
BENCH_LIB = os.path.join(PKG, "libdsa_bench.so")
OBJ_DIR = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wno-unused-result", "-Wno-unused-value",
    # packed fp32 VALU ops are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _sources():
    return sorted(glob.glob(os.path.join(HERE, "*.hip")))


def _bench_sources():
    return sorted(glob.glob(os.path.join(HERE, "bench", "*.hip")))


def _deps():
    return (glob.glob(os.path.join(HERE, "*.h")) + glob.glob(os.path.join(os.path.dirname(PKG), "include", "*.h"))
            + [os.path.join(HERE, "mla_bwd.hip")])          # csrc/bench/bwd_profile.hip includes it


def _compile(src, force):
    prefix = "bench_" if os.path.basename(os.path.dirname(src)) == "bench" else ""
    obj = os.path.join(OBJ_DIR, prefix + os.path.basename(src)[:-4] + ".o")
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
    srcs, bench_srcs = _sources(), _bench_sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as ex:
        results = list(ex.map(lambda s: _compile(s, force), srcs + bench_srcs))
    objs = [o for o, _ in results[:len(srcs)]]
    bench_objs = [o for o, _ in results[len(srcs):]] + [os.path.join(OBJ_DIR, "api.o")]
    for _, log in results:
        if verbose and log.strip():
            print(log)
    for lib, members in ((LIB, objs), (BENCH_LIB, bench_objs)):
        newest = max(os.path.getmtime(o) for o in members)
        if force or not os.path.exists(lib) or os.path.getmtime(lib) < newest:
            cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + members
            res = subprocess.run(cmd, capture_output=True, text=True)
            if res.returncode != 0:
                raise RuntimeError("link failed:\n" + res.stdout + res.stderr)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
