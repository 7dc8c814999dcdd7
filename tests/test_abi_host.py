"""The C ABI from a compiled caller: tests/abi_host/host_check.cpp binds include/electrock_moe.h from C++ over the
HIP runtime, with no Python and no torch in its process, and checks the layer against its own float restatement."""
import os
import subprocess

import pytest

from tests.abi_host import build_host_check as B


def test_host_check_compiles_and_links_against_the_library():
    path = B.build()
    assert os.access(path, os.X_OK)
    needed = subprocess.run(["readelf", "-d", path], stdout=subprocess.PIPE, text=True).stdout
    assert "libelectrock_moe.so" in needed and "torch" not in needed


@pytest.mark.gpu
def test_host_check_runs_the_layer_without_python():
    if not os.path.exists(B.BINARY):
        B.build()
    print("[gpu-case] host_check binary", flush=True)
    proc = subprocess.run([B.BINARY], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout
    assert proc.stdout.strip().endswith("host_check ok")
