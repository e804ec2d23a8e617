"""Builds libh2o4gpu_kmeans_hip.so for gfx950 with hipcc, in-tree."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libh2o4gpu_kmeans_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["engine.hip", "assign_kernels.hip", "longrow_kernels.hip", "update_kernels.hip", "seed_kernels.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-munsafe-fp-atomics", "-pthread",
    # packed-FP32 VALU forms stay off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-result",
]


def build(verbose=False, jobs=4):
    """Compile every .hip source to an object (in parallel) and link the shared library."""
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        while sum(p.poll() is None for _, p in procs) >= jobs:
            procs[0][1].wait()
    failed = False
    for src, p in procs:
        out = p.communicate()[0].decode()
        lines = [l for l in out.splitlines()
                 if "packed-fp32-ops" not in l and "is not a recognized feature" not in l]
        if p.returncode != 0:
            failed = True
            print("\n".join(lines), file=sys.stderr)
        elif verbose and lines:
            print("\n".join(lines))
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-pthread", "-o", LIB_PATH] + objs
    subprocess.check_call(cmd)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
