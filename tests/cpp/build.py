"""Builds the C++ host-layer test driver (tests/cpp/bin/host_api_test) with g++ against the
in-tree header and shared library."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
BIN = os.path.join(HERE, "bin", "host_api_test")


def build():
    os.makedirs(os.path.dirname(BIN), exist_ok=True)
    cmd = ["g++", "-std=c++14", "-O1", "-Wall", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "phoenix_core_amd", "include"), os.path.join(HERE, "host_api_test.cc"), "-o", BIN,
           "-L", os.path.join(ROOT, "phoenix_core_amd", "lib"), "-lphx_qconv",
           "-Wl,-rpath,$ORIGIN/../../../phoenix_core_amd/lib"]
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return BIN


if __name__ == "__main__":
    build()
