"""Compiles host_check.cpp (a C++ caller of the C ABI, no Python in the process) next to its source.  The binary
finds the library through a path relative to itself, so the tree can be moved as a whole."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SOURCE = os.path.join(HERE, "host_check.cpp")
BINARY = os.path.join(HERE, "host_check")


def build() -> str:
    if ROOT not in sys.path:
        sys.path.insert(0, ROOT)
    from electrock_infer_amd import _build
    if not os.path.exists(_build.LIB_PATH):
        raise RuntimeError("build libelectrock_moe.so first")
    cmd = [_build.hipcc_path(), "-O2", "-std=c++17", "-Wall", SOURCE, "-o", BINARY + ".tmp",
           "-L", _build.LIB_DIR, "-lelectrock_moe", "-Wl,-rpath,$ORIGIN/../../electrock_infer_amd/lib"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed on host_check.cpp:\n" + proc.stdout)
    os.replace(BINARY + ".tmp", BINARY)
    return BINARY


if __name__ == "__main__":
    print(build())
