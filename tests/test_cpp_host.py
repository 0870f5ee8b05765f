"""The C++20 host layer (tinytensor_amd/host/tt_amd.h) and its tests, which restate the reference's own
tests/test_matmul.cpp and tests/test_conv.cpp against the AMD device.  The executables are plain g++ programs over
the C ABI; they are built by __graft_entry__.build() (or on demand here) and run on the GPU box."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")
BINARIES = ["test_matmul_amd", "test_conv_amd", "test_ops_amd"]
# The reference-side adapter (host/adapter/.../backend_amd.cpp) compiled against the reference's own backend_base.h with
# the functional stand-ins of tests/cpp/tt_standin/ for the <tt/...> headers, and driven through a BackendBase reference.
# It is built where the reference tree is present (tests/cpp/Makefile); the GPU box runs the executable built beforehand.
ADAPTER_BINARY = "test_adapter_amd"
REFERENCE_HEADER = "/root/reference/tinytensor/tensor/backend_base.h"


def ensure_built():
    wanted = BINARIES + ([ADAPTER_BINARY] if os.path.exists(REFERENCE_HEADER) else [])
    if not all(os.path.exists(os.path.join(CPP, b)) for b in wanted):
        subprocess.run(["make", "-C", CPP], check=True, capture_output=True)


def test_cpp_tests_build_and_list():
    ensure_built()
    for b in BINARIES + ([ADAPTER_BINARY] if os.path.exists(os.path.join(CPP, ADAPTER_BINARY)) else []):
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


@pytest.mark.gpu
def test_reference_side_adapter_runs_on_gpu_through_backend_base():
    """backend_amd.cpp as an object, every call through `const BackendBase &` (tests/cpp/test_adapter_amd.cpp)."""
    ensure_built()
    path = os.path.join(CPP, ADAPTER_BINARY)
    assert os.path.exists(path), "tests/cpp/test_adapter_amd was not built (it needs the reference tree at build time)"
    proc = subprocess.run([path], capture_output=True, text=True, timeout=110)
    print(proc.stdout[-3000:], proc.stderr[-2000:])
    assert proc.returncode == 0, proc.stdout[-3000:]
    assert "0 failure(s)" in proc.stdout
