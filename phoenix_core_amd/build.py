"""Compiles the HIP sources of the engine for gfx950 into phoenix_core_amd/lib/libphx_qconv.so.

Run as `python -m phoenix_core_amd.build`; hipcc cross-compiles without a GPU present."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libphx_qconv.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed fp32 VALU forms are kept out of the device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def build(verbose=True, extra_flags=()):
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [HIPCC] + FLAGS + list(extra_flags) + sources() + ["-o", LIB_PATH]
    if verbose:
        print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if verbose and out.strip():
        print(out, flush=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    return LIB_PATH


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
