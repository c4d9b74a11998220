"""Build recipe for libmoe_hip.so (hipcc, gfx950 only, no torch headers involved).

    python torch-tpu_amd/build.py

The library lands next to this file so that it travels with the source tree.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmoe_hip.so")
SOURCES = ["route.hip", "permute.hip", "quant_reduce.hip", "gemm_fp8.hip", "dense_small.hip", "decode_prep.hip", "router_front.hip",
           "probe.hip", "capi.hip"]
# packed fp32 VALU ops are switched off for every kernel in this library
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build(verbose=True, extra_flags=()):
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for s in SOURCES:
        obj = os.path.join(HERE, "build", s.replace(".hip", ".o"))
        cmd = [hipcc(), *FLAGS, *extra_flags, "-c", os.path.join(CSRC, s), "-o", obj]
        procs.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for s, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "is not a recognized feature for this target" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {s}:\n{out}")
        if verbose and out.strip():
            print(out)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
