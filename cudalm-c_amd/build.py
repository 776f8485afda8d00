"""Compiles libqlmx.so (hand-written HIP for gfx950 behind the C ABI of include/qlmx.h) in-tree.

    python cudalm-c_amd/build.py            # or: build_all() from __graft_entry__.build()

hipcc cross-compiles without a GPU. Flags: no FMA contraction (the integer optimizer is bit-exact
against a CPU build compiled the same way) and no packed-fp32 VALU forms.

The packed-fp32 switch is a target feature of the gfx950 device pass. hipcc hands -Xclang options to its
x86 host pass as well, which does not know the feature and says so once per include ("is not a recognized
feature for this target (ignoring feature)"). That line is dropped from the build output only after the
build has shown that it cannot come from the device pass: a device-only probe compile must accept the
feature without a word, and the device assembly of every source (kept by -save-temps) must be free of
v_pk_add_f32 / v_pk_mul_f32 / v_pk_fma_f32. Either check failing stops the build.
"""
import glob
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libqlmx.so")
HOST_LIB = os.path.join(HERE, "libqlmx_host.so")
ARCH = "gfx950"

HIP_SOURCES = ["qlmx_runtime.hip", "qlmx_step.hip", "qlmx_codec.hip", "qlmx_gemm_common.hip",
               "qlmx_gemm_f32.hip", "qlmx_gemm_mfma.hip", "qlmx_gemm_nt_lds.hip", "qlmx_gemm_tn_lds.hip", "qlmx_gemm_bwd.hip", "qlmx_gemm_nn_lds.hip", "qlmx_gemm_nn_h.hip", "qlmx_gemv.hip", "qlmx_gemm_api.hip", "qlmx_glue.hip", "qlmx_q4n.hip"]
HIP_FLAGS = ["-O3", "--offload-arch=" + ARCH, "-std=c++17", "-fPIC", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]   # = PK_FLAGS, spelled out


HOST_PASS_NOTE = "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)"
PACKED_F32 = re.compile(r"\bv_pk_(add|mul|fma)_f32\b")
PK_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _without_host_pass_note(text):
    return "\n".join(l for l in text.splitlines() if l.strip() != HOST_PASS_NOTE)


def _run(cmd):
    print("+ " + " ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = _without_host_pass_note(p.stdout)
    if out.strip():
        print(out)
    if p.returncode != 0:
        raise RuntimeError("command failed (%d): %s" % (p.returncode, " ".join(cmd)))


def probe_packed_fp32_switch(hipcc):
    """The device pass alone, on a kernel that becomes v_pk_fma_f32 / v_pk_add_f32 by default: with the switch it
    must compile silently (the feature is known to gfx950) and contain no packed-fp32 instruction, without it
    the same source must contain some (so the check can fail)."""
    src = ("#include <hip/hip_runtime.h>\n"
           "__global__ void k(float2 *a, const float2 *b, const float2 *c){ int i = threadIdx.x; float2 x = a[i], y = b[i], z = c[i];\n"
           "  x.x = x.x * y.x + z.x; x.y = x.y * y.y + z.y; x.x += y.x; x.y += y.y; a[i] = x; }\n")
    with tempfile.TemporaryDirectory() as td:
        f = os.path.join(td, "probe.hip")
        open(f, "w").write(src)
        res = {}
        for tag, extra in (("off", PK_FLAGS), ("default", [])):
            out = os.path.join(td, tag + ".s")
            p = subprocess.run([hipcc, "-O3", "--offload-arch=" + ARCH, "--cuda-device-only", "-S", "-Wno-unused-command-line-argument"] + extra + [f, "-o", out],
                               stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
            if p.returncode != 0:
                raise RuntimeError("packed-fp32 probe did not compile:\n" + p.stdout)
            res[tag] = (p.stdout, len(PACKED_F32.findall(open(out).read())))
    if "not a recognized feature" in res["off"][0]:
        raise RuntimeError("the gfx950 device pass rejects -packed-fp32-ops:\n" + res["off"][0])
    if res["off"][1] != 0 or res["default"][1] == 0:
        raise RuntimeError("packed-fp32 probe: %d packed instructions with the switch (want 0), %d without (want > 0)"
                           % (res["off"][1], res["default"][1]))
    print("packed-fp32 switch: accepted by the gfx950 pass; probe kernel has %d packed fp32 instructions without it, 0 with it"
          % res["default"][1], flush=True)


def check_device_asm(objdir):
    """every source's gfx950 assembly (kept by -save-temps=obj) must be free of packed fp32 arithmetic; the
    intermediate files are removed afterwards"""
    bad = []
    asm = glob.glob(os.path.join(objdir, "*-hip-amdgcn-amd-amdhsa-" + ARCH + ".s"))
    for f in asm:
        n = len(PACKED_F32.findall(open(f).read()))
        if n:
            bad.append("%s: %d" % (os.path.basename(f), n))
    for pat in ("*.hipi", "*.bc", "*.s", "*.out", "*.resolution.txt", "*.hipfb", "*-hip-amdgcn-amd-amdhsa-*.o"):
        for f in glob.glob(os.path.join(objdir, pat)):
            os.remove(f)
    if bad:
        raise RuntimeError("packed fp32 instructions in device code: " + ", ".join(bad))
    if len(asm) == 0:
        raise RuntimeError("no device assembly was kept: the packed-fp32 check did not run")
    print("device assembly of %d sources: no v_pk_add_f32 / v_pk_mul_f32 / v_pk_fma_f32" % len(asm), flush=True)


def build_all(jobs=8):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        hipcc = "hipcc"
    probe_packed_fp32_switch(hipcc)
    srcs = [os.path.join(CSRC, s) for s in HIP_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = []
    procs = []
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    for s in srcs:
        o = os.path.join(objdir, os.path.basename(s) + ".o")
        objs.append(o)
        cmd = [hipcc] + HIP_FLAGS + ["-save-temps=obj", "-c", s, "-o", o]
        print("+ " + " ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    check_device_asm(objdir)
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
        out = _without_host_pass_note(out)
        if out.strip():
            print(out)
        if p.returncode != 0:
            raise RuntimeError("command failed (%d): %s" % (p.returncode, " ".join(cmd)))


if __name__ == "__main__":
    build_all()
    print("built", LIB)
