"""Compiles libqlmx.so (hand-written HIP for gfx950 behind the C ABI of include/qlmx.h) in-tree.

    python cudalm-c_amd/build.py            # or: build_all() from __graft_entry__.build()

hipcc cross-compiles without a GPU. Flags: no FMA contraction (the integer optimizer is bit-exact
against a CPU build compiled the same way) and no packed-fp32 VALU forms.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libqlmx.so")
HOST_LIB = os.path.join(HERE, "libqlmx_host.so")
ARCH = "gfx950"

HIP_SOURCES = ["qlmx_runtime.hip", "qlmx_step.hip", "qlmx_codec.hip", "qlmx_gemm_common.hip",
               "qlmx_gemm_f32.hip", "qlmx_gemm_mfma.hip", "qlmx_gemm_nt_lds.hip", "qlmx_gemm_tn_lds.hip", "qlmx_gemm_nn_lds.hip", "qlmx_gemv.hip", "qlmx_gemm_api.hip", "qlmx_glue.hip", "qlmx_q4n.hip"]
HIP_FLAGS = ["-O3", "--offload-arch=" + ARCH, "-std=c++17", "-fPIC", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def _run(cmd):
    print("+ " + " ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if out.strip():
        print(out)
    if p.returncode != 0:
        raise RuntimeError("command failed (%d): %s" % (p.returncode, " ".join(cmd)))


def build_all(jobs=8):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        hipcc = "hipcc"
    srcs = [os.path.join(CSRC, s) for s in HIP_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = []
    procs = []
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    for s in srcs:
        o = os.path.join(objdir, os.path.basename(s) + ".o")
        objs.append(o)
        cmd = [hipcc] + HIP_FLAGS + ["-c", s, "-o", o]
        print("+ " + " ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    _run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC"] + objs + ["-o", LIB])
    host_src = os.path.join(HERE, "host", "qlm_host.cpp")
    if os.path.exists(host_src):
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-I", os.path.join(HERE, "..", "include"),
              host_src, "-o", HOST_LIB, "-L", HERE, "-lqlmx", "-Wl,-rpath,$ORIGIN"])
        _run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-I", os.path.join(HERE, "..", "include"),
              os.path.join(HERE, "host", "selftest.cpp"), "-o", os.path.join(HERE, "qlm_selftest"),
              "-L", HERE, "-lqlmx_host", "-lqlmx", "-Wl,-rpath,$ORIGIN"])
    return LIB


def _drain(procs):
    while procs:
        cmd, p = procs.pop(0)
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "is not a recognized feature for this target" not in l)
        if out.strip():
            print(out)
        if p.returncode != 0:
            raise RuntimeError("command failed (%d): %s" % (p.returncode, " ".join(cmd)))


if __name__ == "__main__":
    build_all()
    print("built", LIB)
