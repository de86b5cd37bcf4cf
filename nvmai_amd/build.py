"""Builds libnvmai_hip.so in-tree with hipcc for gfx950."""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libnvmai_hip.so")

FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function",
         # "#pragma unroll" on loops whose trip count is a template parameter: the instantiations that take
         # the count at run time cannot unroll, and say so once per loop
         "-Wno-pass-failed"]


def build(verbose=False, jobs=8):
    """Compile every .hip file under csrc/ and link them into one shared library."""
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs, procs = [], []
    for src in srcs:
        obj = src[:-4] + ".o"
        objs.append(obj)
        cmd = ["hipcc", *FLAGS, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        if len(procs) >= jobs:
            _wait(procs)
    _wait(procs)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    subprocess.run(cmd, check=True)
    return LIB


def _wait(procs):
    while procs:
        src, proc = procs.pop(0)
        out = proc.communicate()[0].decode()
        # the host pass does not know the packed-fp32 feature flag and says so
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if out.strip():
            print(out, file=sys.stderr)


if __name__ == "__main__":
    print(build(verbose=True))
