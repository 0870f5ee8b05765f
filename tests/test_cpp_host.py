"""The C++20 host layer (tinytensor_amd/host/tt_amd.h) and its tests, which restate the reference's own
tests/test_matmul.cpp and tests/test_conv.cpp against the AMD device.  The executables are plain g++ programs over
the C ABI; they are built by __graft_entry__.build() (or on demand here) and run on the GPU box."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")
BINARIES = ["test_matmul_amd", "test_conv_amd", "test_ops_amd"]


def ensure_built():
    if not all(os.path.exists(os.path.join(CPP, b)) for b in BINARIES):
        subprocess.run(["make", "-C", CPP], check=True, capture_output=True)


def test_cpp_tests_build_and_list():
    ensure_built()
    for b in BINARIES:
        out = subprocess.run([os.path.join(CPP, b), "--list"], check=True, capture_output=True, text=True).stdout
        assert len(out.strip().splitlines()) >= 2


@pytest.mark.gpu
@pytest.mark.parametrize("binary", BINARIES)
def test_cpp_host_layer_on_gpu(binary):
    ensure_built()
    proc = subprocess.run([os.path.join(CPP, binary)], capture_output=True, text=True, timeout=110)
    print(proc.stdout[-3000:], proc.stderr[-2000:])
    assert proc.returncode == 0, proc.stdout[-3000:]
    assert "0 failure(s)" in proc.stdout
