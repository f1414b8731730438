"""Compile the gfx950 HIP library in-tree with hipcc.

`python -m blitz_scale_amd.build` writes blitz_scale_amd/lib/libbz_hip.so.  The library is plain
HIP + a C ABI (include/bz_hip.h); it does not link against torch.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libbz_hip.so")

SOURCES = [
    "bz_decode_plan.hip",
    "bz_decode.hip",
    "bz_decode_mfma.hip",
    "bz_prefill.hip",
    "bz_page.hip",
    "bz_elementwise.hip",
    "bz_sampler.hip",
    "bz_wire.hip",
    "bz_host.hip",
]

# packed fp32 VALU forms are kept off for every device compile of this library
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    "-Wno-inline-asm",
]


# bz_decode_mfma.hip: the leading pointers of a kernel's argument list arrive in registers with the wave
# (kernel-argument preload of gfx950), which lets the decode kernel ask for its slot head, and the finishing kernel
# of the decode step for its unit record, while the other arguments are still being fetched: one scalar round trip
# less at the head of each.  A kernel whose first argument is a struct is unaffected.
EXTRA_FLAGS = {
    "bz_decode_mfma.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=4"],
}


def hipcc():
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def build(verbose=True, jobs=8):
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            continue
        obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), "-I", os.path.join(ROOT, "include"),
               "-I", os.path.join(HERE, "cpp", "kernel"),
               "-c", path, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


PROBE_SRC = os.path.join(HERE, "probes", "mfma_ceiling.hip")
PROBE_BIN = os.path.join(HERE, "probes", "mfma_ceiling")


def build_probes(verbose=True):
    """The stand-alone measurement program behind `bench.py --workload MFMA_CEILING` (no part of the library)."""
    cmd = [hipcc(), *[f for f in HIPCC_FLAGS if f != "-fPIC"], PROBE_SRC, "-o", PROBE_BIN]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    text = "\n".join(l for l in out.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed on the probe:\n" + text)
    return PROBE_BIN


def _drain(procs):
    failed = []
    for src, p in procs:
        out, _ = p.communicate()
        # the host pass does not know the packed-fp32 target feature and says so: harmless
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed.append((src, out))
        elif out.strip():
            print(out)
    procs.clear()
    if failed:
        for src, out in failed:
            sys.stderr.write(f"--- {src} failed ---\n{out}\n")
        raise RuntimeError("hipcc failed for: " + ", ".join(s for s, _ in failed))


if __name__ == "__main__":
    print(build())
