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


def _compile_one(job):
    src, obj, flags = job
    cmd = [HIPCC] + flags + ["-c", src, "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    return src, proc.returncode, out


def build(verbose=True, extra_flags=()):
    """Compile every csrc/*.hip to an object (in parallel) and link libphx_qconv.so."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB_DIR, exist_ok=True)
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    flags = [f for f in FLAGS if f != "-shared"] + list(extra_flags)
    jobs = [(src, os.path.join(objdir, os.path.basename(src)[:-4] + ".o"), flags) for src in sources()]
    if verbose:
        print("+ %s %s -c {%s}" % (HIPCC, " ".join(flags), ", ".join(os.path.basename(j[0]) for j in jobs)), flush=True)
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        results = list(pool.map(_compile_one, jobs))
    for src, rc, out in results:
        if verbose and out.strip():
            print(out, flush=True)
        if rc != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
    link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + [j[1] for j in jobs] + ["-o", LIB_PATH]
    if verbose:
        print("+", " ".join(link), flush=True)
    proc = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stdout)
    return LIB_PATH


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
