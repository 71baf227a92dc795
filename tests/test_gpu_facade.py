"""Runs the C++ ClusterNet / Matrix test program (tests/cpp/facade_test.cpp) on the GPU box."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "cpp", "facade_test")


@pytest.mark.gpu
def test_facade_program():
    assert os.path.exists(BINARY), "tests/cpp/facade_test is not built (run __graft_entry__.build())"
    proc = subprocess.run([BINARY], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=240)
    print(proc.stdout[-4000:])
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "ALL FACADE TESTS PASSED" in proc.stdout


def test_facade_library_exports_the_reference_api():
    lib = os.path.join(ROOT, "clusternet_amd", "libclusternet.so")
    assert os.path.exists(lib), "libclusternet.so is not built"
    syms = subprocess.run(["nm", "-DC", lib], stdout=subprocess.PIPE, text=True).stdout
    for name in ("ClusterNet::dot(Matrix*, Matrix*)", "ClusterNet::Tdot(Matrix*, Matrix*, Matrix*)",
                 "ClusterNet::dotT(Matrix*, Matrix*, Matrix*)", "ClusterNet::dotMPI(Matrix*, Matrix*)",
                 "ClusterNet::compression_8bit(Matrix*, float)", "ClusterNet::decompression_8bit(Matrix*, float, Matrix*)",
                 "ClusterNet::tick(", "ClusterNet::tock(", "to_gpu(Matrix*)", "to_host(Matrix*)", "empty_char(int, int)",
                 "zeros(int, int)", "checkMatrixOperation("):
        assert name in syms, name
