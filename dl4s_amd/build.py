"""Builds libdl4s_hip.so (and the host-layer library) for gfx950 with hipcc, in-tree.

hipcc cross-compiles without a GPU.  Run as `python -m dl4s_amd.build`.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libdl4s_hip.so")
HOST_LIB = os.path.join(HERE, "libdl4s_host.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    "-Wall", "-Wno-unused-function",
    # keep the compiler from forming packed fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose=False):
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError("no HIP sources under %s" % CSRC)
    objs = []
    procs = []
    for s in srcs:
        o = s[:-4] + ".o"
        objs.append(o)
        cmd = [HIPCC] + [f for f in FLAGS if f != "-shared"] + ["-c", s, "-o", o]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for s, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l or "error" in l)
        if p.returncode != 0:
            failed = True
            sys.stderr.write("FAILED: %s\n%s\n" % (s, out))
        elif verbose and out.strip():
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    build_host(verbose)
    return LIB


def build_host(verbose=False):
    """The C++ host layer (no device code): g++ against the C ABI, linked to libdl4s_hip.so next to it."""
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-o", HOST_LIB,
           os.path.join(HERE, "host", "dl4s_host_capi.cpp"), "-L" + HERE, "-ldl4s_hip", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return HOST_LIB


if __name__ == "__main__":
    print(build(verbose=True))
