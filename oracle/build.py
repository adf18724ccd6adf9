"""TEST INFRASTRUCTURE ONLY -- builds the CPU oracle (oracle/libqoracle.so) with gcc and, when the
reference tree is present, the reference-derived checker oracle/_ref/libref_shim.so from the
reference's own algebras.cc / backend.cc.  Run as `python oracle/build.py` or via build()."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = os.environ.get("PHX_REFERENCE_DIR", "/root/reference")


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_oracle():
    out = os.path.join(HERE, "libqoracle.so")
    _run(["gcc", "-O2", "-fopenmp", "-fno-fast-math", "-ffp-contract=off", "-shared", "-fPIC", "-Wall",
          os.path.join(HERE, "qoracle.c"), "-o", out, "-lm"])
    return out


def build_ref():
    """Compiles the buildable slice of the reference (sign tables, product iterators, Context)."""
    src = os.path.join(REFERENCE, "src")
    if not os.path.isfile(os.path.join(src, "algebras.cc")):
        print("reference tree not present: skipping oracle/_ref", flush=True)
        return None
    outdir = os.path.join(HERE, "_ref")
    os.makedirs(outdir, exist_ok=True)
    out = os.path.join(outdir, "libref_shim.so")
    _run(["g++", "-std=c++14", "-O1", "-w", "-shared", "-fPIC", "-I", src,
          os.path.join(HERE, "ref_shim.cc"),
          os.path.join(src, "algebras.cc"),
          os.path.join(src, "backend", "backend.cc"),
          "-o", out])
    return out


def main():
    build_oracle()
    build_ref()


if __name__ == "__main__":
    sys.exit(main())
