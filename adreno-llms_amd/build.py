"""Builds libmi_linear.so (gfx950 only) in-tree with hipcc.

Usage: python adreno-llms_amd/build.py  (or __graft_entry__.build()).
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libmi_linear.so")
SOURCES = ["runtime.hip", "gemv.hip", "gemm.hip", "argmax.hip", "decode.hip", "probe.hip", "quantize.cpp", "bundle.cpp"]

# -ffp-contract=off: the kernels spell every fused multiply-add as fmaf(); nothing else
# may be fused, or results stop being bit-identical to the reference evaluation order.
# The packed-fp32 feature is switched off for device code on purpose.
COMMON = ["-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Wall", "-Wno-unused-result"]
# (fp32 divide and square root correctly rounded: hipcc's default, spelled out because the
#  decode-step kernels rely on it for bit-identical results)
# (the first 16 dwords of a kernel's arguments arrive in scalar registers with the wavefront instead of
#  being fetched by its first instructions: a launch-bound kernel starts its loads that much earlier;
#  measured on the decode sweep, 331 -> 326 us, and on the whole decode step, 490 -> 475 us)
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-fhip-fp32-correctly-rounded-divide-sqrt", "-mllvm", "-amdgpu-kernarg-preload-count=16"]


def build(verbose=True, extra=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc, *COMMON, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if src.endswith(".hip"):
            cmd[1:1] = DEVICE
        else:
            cmd[1:1] = ["-x", "c++"]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip() and verbose:
            print(out)
        if p.returncode != 0:
            print(f"build of {src} failed", file=sys.stderr)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed")
    link = [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", OUT, *objs, "-lpthread"]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.check_call(link)
    return OUT


if __name__ == "__main__":
    build()
