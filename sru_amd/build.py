"""Builds sru_amd/libsru_amd.so for gfx950 with hipcc.  `python -m sru_amd.build`"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SOURCES = [os.path.join(HERE, "csrc", n)
           for n in ("sru_amd.hip", "scan_f32.hip", "scan_f16.hip", "scan_bf16.hip")]
OUTPUT = os.path.join(HERE, "libsru_amd.so")
OBJ_DIR = os.path.join(HERE, "csrc", "build")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-FP32 instructions stay off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"),
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature and says so: harmless
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if out and (verbose or proc.returncode):
        print(out, flush=True)
    if proc.returncode:
        raise RuntimeError("hipcc failed: " + " ".join(cmd))


def build(verbose=True, output=OUTPUT, defines=()):
    """Compiles every translation unit (in parallel) and links the shared library.

    `defines` (e.g. ["SRU_AMD_F32_COLS=2"]) and `output` serve tuning builds."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    tag = "".join(c if c.isalnum() else "_" for c in "_".join(defines))
    obj_dir = os.path.join(OBJ_DIR, tag) if tag else OBJ_DIR
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o") for src in SOURCES]
    extra = ["-D" + d for d in defines]
    jobs = [[hipcc] + HIPCC_FLAGS + extra + ["-c", src, "-o", obj] for src, obj in zip(SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=4) as pool:
        list(pool.map(lambda cmd: _run(cmd, verbose), jobs))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", output], verbose)
    return output


if __name__ == "__main__":
    build()
    sys.exit(0)
