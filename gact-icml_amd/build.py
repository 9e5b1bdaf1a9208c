"""Build libgact_hip.so (the C-ABI library of HIP kernels) and libgact_probe.so (compute-free traffic probes that
bench.py measures beside the kernels) for gfx950 with hipcc.

    python gact-icml_amd/build.py            # build if the sources are newer than the library
    python gact-icml_amd/build.py --force

hipcc cross-compiles for gfx950 without a GPU present.  The library lands inside the Python
package (gact/lib/) so that it travels with the source tree.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "csrc", "gact_hip.hip")
PROBE_SRC = os.path.join(HERE, "csrc", "stream_probe.hip")   # compute-free traffic probes for bench.py
HDR = os.path.join(ROOT, "include", "gact_hip.h")
OUT_DIR = os.path.join(HERE, "gact", "lib")
OUT = os.path.join(OUT_DIR, "libgact_hip.so")
PROBE_OUT = os.path.join(OUT_DIR, "libgact_probe.so")

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # every floating-point operation in the kernels is meant literally (the one FMA is spelled out)
    "-ffp-contract=off",
    # keep the compiler from forming packed-FP32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first 16 dwords of a kernel's arguments arrive in scalar registers with the wave (gfx950 preloads them) instead
    # of through a load that every wave waits for before it can ask for data: dequantize of a 16 MB float tensor
    # 4.40 -> 4.22 us, of a 34 MB half tensor 9.15 -> 9.02, large tensors 0.5-1 %.  The quantize kernels, which lose up
    # to 0.5 % by it, take a structure as their first argument and so stay as they were.
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall",
    "-Wno-unused-command-line-argument",
]


def hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC)")


def up_to_date():
    if not os.path.exists(OUT) or not os.path.exists(PROBE_OUT):
        return False
    t = min(os.path.getmtime(OUT), os.path.getmtime(PROBE_OUT))
    return all(os.path.getmtime(p) <= t for p in (SRC, PROBE_SRC, HDR, os.path.abspath(__file__)))


def build(force=False, extra=()):
    if not force and up_to_date():
        return OUT
    os.makedirs(OUT_DIR, exist_ok=True)
    cmd = [hipcc()] + HIPCC_FLAGS + list(extra) + ["-I", os.path.join(ROOT, "include"), "-o", OUT, SRC]
    subprocess.run(cmd, check=True)
    subprocess.run([hipcc()] + HIPCC_FLAGS + ["-o", PROBE_OUT, PROBE_SRC], check=True)
    return OUT


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
