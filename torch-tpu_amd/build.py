"""Build recipe for libmoe_hip.so (hipcc, gfx950 only, no torch headers involved) and, beside it,
libmy_ops_torch.so (g++ against the torch headers, no device code: the C++ operator registration that forwards to
the C ABI) and libmoe_bench_probe.so (the benchmark's read probe, kept out of the product library and loaded by
bench.py only).

    python torch-tpu_amd/build.py

The libraries land next to this file so that they travel with the source tree.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmoe_hip.so")
PROBE_LIB = os.path.join(HERE, "libmoe_bench_probe.so")
SOURCES = ["route.hip", "permute.hip", "quant_reduce.hip", "gemm_fp8.hip", "dense_small.hip", "decode_prep.hip", "router_front.hip",
           "capi.hip"]
PROBE_SOURCES = ["probe.hip"]
SHIM_LIB = os.path.join(HERE, "libmy_ops_torch.so")
SHIM_SOURCE = "my_ops.cpp"
# packed fp32 VALU ops are switched off for every kernel in this library
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build_shim(verbose=True):
    """csrc/my_ops.cpp -> libmy_ops_torch.so: TORCH_LIBRARY(my_ops, ...) on top of libmoe_hip.so, plain host C++."""
    import torch
    tdir = os.path.dirname(os.path.abspath(torch.__file__))
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unknown-pragmas", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I" + os.path.join(tdir, "include"), "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           "-I/opt/rocm/include", os.path.join(CSRC, SHIM_SOURCE), "-o", SHIM_LIB,
           "-L" + os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-lamdhip64", "-L" + HERE, "-lmoe_hip",
           "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the operator registration failed:\n" + r.stdout)
    if verbose:
        print("built", SHIM_LIB)
    return SHIM_LIB


def build(verbose=True, extra_flags=(), shim=True):
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for s in SOURCES + PROBE_SOURCES:
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
    n = len(SOURCES)
    for lib, lib_objs in ((LIB, objs[:n]), (PROBE_LIB, objs[n:])):
        cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *lib_objs, "-o", lib]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stdout)
        if verbose:
            print("built", lib)
    if shim:
        build_shim(verbose)
    return LIB


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
