"""Builds libmarlin_amd.so (HIP kernels + C ABI) and libmarlin_amd_probe.so (the
measurement probes of the benchmark) in-tree for gfx950."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmarlin_amd.so")
PROBE_LIB = os.path.join(HERE, "libmarlin_amd_probe.so")
# source -> extra flags.  The prefill kernel keeps its 128 accumulator registers
# in ordinary VGPRs (it fits in 256), which spares the AGPR copy traffic the
# default register split produces around every MFMA.
SOURCES = {
    "marlin_host.hip": [],
    "scratch_pool.hip": [],
    "w4a16_stream.hip": [],
    "w4a16_strip.hip": [],
    "w4a16_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "w4a16_prefill_wide.hip": [],
    "f16_streamk.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I", os.path.join(HERE, "build"),
    # packed fp32 arithmetic stays off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)


def build_library(verbose=False):
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    # the assembly statements of the four-wave prefill kernel (prologue, main
    # loop and accumulator hand-over with fixed registers) are written by a
    # generator; w4a16_prefill_wide.hip includes them from the build directory
    _run([sys.executable, os.path.join(CSRC, "gen_prefill_wide.py"), objdir], verbose)
    objs = []
    for src, extra in SOURCES.items():
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        _run([HIPCC] + FLAGS + extra + ["-c", "-o", obj, os.path.join(CSRC, src)], verbose)
        objs.append(obj)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs, verbose)
    # the probes: a library of their own that asks the first one for its plans
    obj = os.path.join(objdir, "w4a16_probe.o")
    _run([HIPCC] + FLAGS + ["-c", "-o", obj, os.path.join(CSRC, "w4a16_probe.hip")], verbose)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROBE_LIB, obj, "-L", HERE,
          "-lmarlin_amd", "-Wl,-rpath,$ORIGIN"], verbose)
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True))
