"""Builds sru_amd/libsru_amd.so for gfx950 with hipcc.  `python -m sru_amd.build`"""
import json
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SOURCES = [os.path.join(HERE, "csrc", n)
           for n in ("sru_amd.hip", "sru_norm.hip", "scan_f32_fwd.hip", "scan_f32_bwd.hip", "scan_f16_fwd.hip",
                     "scan_f16_bwd.hip", "scan_bf16_fwd.hip", "scan_bf16_bwd.hip", "scan_f64.hip")]
OUTPUT = os.path.join(HERE, "libsru_amd.so")
OBJ_DIR = os.path.join(HERE, "csrc", "build")
SERVE_FORWARD = os.path.join(HERE, "serve_forward")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-FP32 instructions stay off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"),
]


# A kernel whose register ring or chunk ends up in scratch memory runs several times slower
# with unchanged results, so the build checks the compiler's resource report and refuses any
# kernel that keeps anything in scratch memory.
MAX_SCRATCH_BYTES = 0
_REMARK = re.compile(r"remark: .*?(Function Name: (?P<name>\S+)|ScratchSize \[bytes/lane\]: (?P<scratch>\d+)"
                     r"|VGPRs: (?P<vgprs>\d+))")


def _run(cmd, verbose):
    """Runs one hipcc command; returns {kernel: (vgprs, scratch_bytes)} from its resource remarks."""
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    usage, name, vgprs = {}, None, None
    other = []
    in_remark = False
    for line in proc.stdout.splitlines():
        if in_remark and re.match(r"\s*(\d+)?\s*\|", line):
            continue            # source excerpt under a remark
        in_remark = "remark:" in line
        m = _REMARK.search(line)
        if m:
            if m.group("name"):
                name, vgprs = m.group("name"), None
            elif m.group("vgprs") and " VGPRs:" in line:
                vgprs = int(m.group("vgprs"))
            elif m.group("scratch") is not None and name:
                usage[name] = (vgprs, int(m.group("scratch")))
            continue
        # the host pass does not know the device-only target feature and says so: harmless
        if ("remark:" in line or "packed-fp32-ops" in line or not line.strip()
                or line.startswith("In file included from")):
            continue
        other.append(line)
    if other and (verbose or proc.returncode):
        print("\n".join(other), flush=True)
    if proc.returncode:
        raise RuntimeError("hipcc failed: " + " ".join(cmd))
    return usage


def build(verbose=True, output=OUTPUT, defines=(), max_scratch_bytes=MAX_SCRATCH_BYTES):
    """Compiles every translation unit (in parallel) and links the shared library.

    `defines` (e.g. ["SRU_AMD_PAIR_BELOW=131072"]), `output` and `max_scratch_bytes` serve tuning builds."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    tag = "".join(c if c.isalnum() else "_" for c in "_".join(defines))
    obj_dir = os.path.join(OBJ_DIR, tag) if tag else OBJ_DIR
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o") for src in SOURCES]
    extra = ["-D" + d for d in defines]
    jobs = [[hipcc] + HIPCC_FLAGS + extra + ["-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", obj]
            for src, obj in zip(SOURCES, objs)]
    usage = {}
    with ThreadPoolExecutor(max_workers=len(jobs)) as pool:
        for part in pool.map(lambda cmd: _run(cmd, verbose), jobs):
            usage.update(part)
    with open(os.path.join(obj_dir, "resource_usage.json"), "w") as f:
        json.dump({k: {"vgprs": v[0], "scratch_bytes": v[1]} for k, v in sorted(usage.items())}, f, indent=1)
    spilled = {k: v[1] for k, v in usage.items() if v[1] > max_scratch_bytes}
    if spilled:
        raise RuntimeError(f"{len(spilled)} kernels keep more than {max_scratch_bytes} bytes per lane in "
                           f"scratch memory, e.g. {sorted(spilled.items(), key=lambda kv: -kv[1])[:3]}")
    if verbose:
        print(f"{len(usage)} kernels, largest scratch {max([v[1] for v in usage.values()] or [0])} bytes/lane, "
              f"largest VGPR count {max([v[0] or 0 for v in usage.values()] or [0])}", flush=True)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", output], verbose)
    if output == OUTPUT:
        build_serve_forward(verbose)
    return output


def build_serve_forward(verbose=True):
    """Compiles csrc/serve_forward.cpp, a caller of the C ABI without Python or torch, with the
    host compiler against the library just built (found at run time next to the program)."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-D__HIP_PLATFORM_AMD__",
           "-I" + os.path.join(rocm, "include"), "-I" + os.path.join(ROOT, "include"),
           os.path.join(HERE, "csrc", "serve_forward.cpp"), "-L" + HERE, "-lsru_amd",
           "-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath,$ORIGIN",
           "-Wl,-rpath," + os.path.join(rocm, "lib"), "-o", SERVE_FORWARD]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode:
        print(proc.stdout, flush=True)
        raise RuntimeError("host compiler failed: " + " ".join(cmd))
    return SERVE_FORWARD


if __name__ == "__main__":
    build()
    sys.exit(0)
