"""Builds trak_amd/libtrakhip.so from trak_amd/csrc/*.hip with hipcc for gfx950.

Run as `python -m trak_amd.build`.  hipcc cross-compiles, so no GPU is needed to build.
`python -m trak_amd.build --diag` also builds libtrakhip_diag.so, the measurement aid behind
`bench.py --only mfma_rate` (not part of the product library; bench.py builds it when it is asked for).
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtrakhip.so")
DIAG_LIB = os.path.join(HERE, "libtrakhip_diag.so")  # measurement aid for bench.py, not the product ABI
DIAG_SOURCES = ["mfma_rate.hip"]
SOURCES = ["capi.hip", "project.hip", "gemm.hip", "spd.hip", "store.hip", "gemm_split.hip"]
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# hipcc's host pass does not know the device-only target feature and says so once per source: noise
_KNOWN_NOISE = "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)"


def _without_noise(text):
    return "\n".join(l for l in text.splitlines() if l.strip() != _KNOWN_NOISE)


def build(verbose=True, jobs=4, diag=False):
    """Compile every source to an object (in parallel) and link the shared library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [hipcc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    if diag:
        build_diag(verbose)
    return LIB


def build_diag(verbose=True):
    """The measurement aid (a loop of nothing but MFMAs, for `bench.py --only mfma_rate`)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *FLAGS, "-shared", "-o", DIAG_LIB, *[os.path.join(CSRC, s) for s in DIAG_SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    text = _without_noise(out.stdout.decode(errors="replace"))
    if text.strip():
        print(text)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed on the measurement aid")
    return DIAG_LIB


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        text = _without_noise(out.decode(errors="replace"))
        if text.strip():
            print(text)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}")


if __name__ == "__main__":
    build(diag="--diag" in sys.argv[1:])
    print(LIB)
    sys.exit(0)
