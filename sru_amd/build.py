"""Builds sru_amd/libsru_amd.so for gfx950 with hipcc.  `python -m sru_amd.build`"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SOURCES = [os.path.join(HERE, "csrc", "sru_amd.hip")]
OUTPUT = os.path.join(HERE, "libsru_amd.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-FP32 instructions stay off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"),
]


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + SOURCES + ["-o", OUTPUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature and says so: harmless
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if out and (verbose or proc.returncode):
        print(out, flush=True)
    if proc.returncode:
        raise RuntimeError("hipcc failed building libsru_amd.so")
    return OUTPUT


if __name__ == "__main__":
    build()
    sys.exit(0)
