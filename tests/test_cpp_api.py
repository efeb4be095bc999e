"""Runs the C++ programs that use the sycldnn:: drop-in headers
(tests/cpp/*.cpp, built by __graft_entry__.build())."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin")


def _exe(name):
    path = os.path.join(BIN, name)
    if not os.path.exists(path):
        from portdnn_amd import build
        import oracle
        oracle.lib()  # makes sure liboracle.so exists
        build.build_cpp_tests()
    return path


def test_host_api_program():
    """Params, sizes, padding, selectors, workspace sizes and the status codes
    of rejected launches -- no GPU needed."""
    out = subprocess.run([_exe("host_api_test")], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True, timeout=120)
    assert out.returncode == 0, out.stdout
    assert "0 failures" in out.stdout


@pytest.mark.gpu
def test_gpu_api_program():
    """conv2d (every selector, three directions), depthwise, pooling and event
    dependencies through sycldnn::...::launch with backend::HIPBackend."""
    out = subprocess.run([_exe("gpu_api_test")], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True, timeout=300)
    assert out.returncode == 0, out.stdout[-4000:]
    assert "0 failures" in out.stdout
