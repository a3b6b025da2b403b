"""Build libgtm_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m graphtsetlinmachine_amd.build
"""

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = [os.path.join(HERE, "csrc", "gtm_hip.hip")]
OUTPUT = os.path.join(HERE, "libgtm_hip.so")

# -packed-fp32-ops: keep the compiler from forming packed FP32 instructions.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-shared", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


ENCODER_SOURCE = os.path.join(HERE, "csrc", "encode.c")
ENCODER_OUTPUT = os.path.join(HERE, "libgtm_encode.so")


def build_encoder(verbose=True):
    """The host-side property encoder (plain C, OpenMP) that graphs.py loads through ctypes."""
    cmd = [os.environ.get("CC", "gcc"), "-O3", "-fopenmp", "-shared", "-fPIC", "-o", ENCODER_OUTPUT, ENCODER_SOURCE]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("gcc failed:\n" + proc.stdout)
    return ENCODER_OUTPUT


def build(verbose=True):
    build_encoder(verbose)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + ["-o", OUTPUT] + SOURCES
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if verbose and out.strip():
        print(out)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    return OUTPUT


if __name__ == "__main__":
    build()
    sys.exit(0)
