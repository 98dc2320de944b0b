"""Runs the C++ test program of the host mirror classes (cntk_amd/cpp/MatrixQuantizer.h over the C ABI) on the GPU.
The program follows the reference's own unit test (Tests/UnitTests/MathTests/MatrixQuantizerTests.cpp)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "bin", "test_matrix_quantizer")


@pytest.mark.gpu
def test_cpp_matrix_quantizer_suite():
    assert os.path.exists(EXE), "build it first: python -m cntk_amd.build"
    res = subprocess.run([EXE], capture_output=True, text=True, timeout=600)
    print(res.stdout)
    print(res.stderr[-4000:])
    assert res.returncode == 0, "C++ quantizer tests failed"
    assert "GPUMatrix1BitQuantizeFloat has passed" in res.stdout
    assert "QuantizerErrorBehaviour has passed" in res.stdout
    assert "QuantizerBatchEqualsPerMatrix has passed" in res.stdout


def test_cpp_mirror_header_is_self_contained():
    """The mirror header compiles as plain host C++ (no device code, no torch)."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    src = '#include "%s"\nint main() { return sizeof(cntk_amd::QuantizedColumn<float>) == 12 ? 0 : 1; }\n' % os.path.join(
        ROOT, "cntk_amd", "cpp", "MatrixQuantizer.h")
    res = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(rocm, "include"),
                          "-x", "c++", "-"], input=src, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
