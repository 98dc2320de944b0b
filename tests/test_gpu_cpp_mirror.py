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
    assert "GPUMatrix1BitQuantizeDouble has passed" in res.stdout
    assert "QuantizerErrorBehaviour has passed" in res.stdout
    assert "QuantizerBatchEqualsPerMatrix has passed" in res.stdout


@pytest.mark.gpu
def test_cpp_allreduce_aggregator_suite():
    """The aggregator restatement (cntk_amd/cpp/AllReduceDistGradAggregator.h) with K in-process workers."""
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "test_allreduce_aggregator")
    assert os.path.exists(exe), "build it first: python -m cntk_amd.build"
    res = subprocess.run([exe], capture_output=True, text=True, timeout=900)
    print(res.stdout)
    print(res.stderr[-4000:])
    assert res.returncode == 0, "C++ aggregator tests failed"
    for name in ("VariantsBitIdentical", "AgainstOracle", "UnquantizedSelfStripe", "EmptyMinibatchAndReset", "BufferedAggregation"):
        assert "QuantizedAllReduce%s has passed" % name in res.stdout


@pytest.mark.gpu
def test_cpp_distributed_learner_suite():
    """The learner glue (cntk_amd/cpp/QuantizedDataParallelDistributedLearner.h) with K in-process ranks."""
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "test_distributed_learner")
    assert os.path.exists(exe), "build it first: python -m cntk_amd.build"
    res = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    print(res.stdout)
    print(res.stderr[-4000:])
    assert res.returncode == 0, "C++ distributed learner tests failed"
    for name in ("WarmStartThenExactSum", "OneBitUidOrderEmptyAndCheckpoint"):
        assert "DistributedLearner%s has passed" % name in res.stdout


@pytest.mark.gpu
def test_cpp_quantized_communicator_suite():
    """The v2 communicator's call shape (cntk_amd/cpp/QuantizedDistributedCommunicator.h): out-of-place values and residues
    against the aliased form, against the v1 aggregator, float and double by argument type."""
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "test_quantized_communicator")
    assert os.path.exists(exe), "build it first: python -m cntk_amd.build"
    res = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    print(res.stdout)
    print(res.stderr[-4000:])
    assert res.returncode == 0, "C++ communicator tests failed"
    for name in ("OutOfPlaceEqualsAliasedFloat", "OutOfPlaceEqualsAliasedDouble", "EqualsAggregatorAndCallSequence", "TypesAndTrivialCases"):
        assert "CommunicatorSuite/%s has passed" % name in res.stdout


@pytest.mark.gpu
def test_cpp_v2_aggregator_suite():
    """The aggregator over the v2 communicator (cntk_amd/cpp/V2AllReduceDistGradAggregator.h): the v1 aggregator's bytes and
    header, the header sent as doubles, workers without samples, reset, double buffering."""
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "test_v2_aggregator")
    assert os.path.exists(exe), "build it first: python -m cntk_amd.build"
    res = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    print(res.stdout)
    print(res.stderr[-4000:])
    assert res.returncode == 0, "C++ v2 aggregator tests failed"
    for name in ("EqualsV1AggregatorFloat", "EqualsV1AggregatorDouble", "HeaderAsDoubles", "WorkerWithoutSamples", "ResetClearsResidues",
                 "DoubleBuffered"):
        assert "V2AggregatorSuite/%s has passed" % name in res.stdout


@pytest.mark.gpu
def test_cpp_allreduce_timing_program_runs():
    """The all-reduce timing program runs through on a small shape and prints one line per arrangement."""
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "bench_allreduce")
    assert os.path.exists(exe), "build it first: python -m cntk_amd.build"
    res = subprocess.run([exe, "4", "2048", "256", "1", "3"], capture_output=True, text=True, timeout=300)
    print(res.stdout, res.stderr[-2000:])
    assert res.returncode == 0 and res.stdout.count("GB/s") == 4  # one line per arrangement


def test_cpp_mirror_header_is_self_contained():
    """The mirror header compiles as plain host C++ (no device code, no torch)."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    src = '#include "%s"\nint main() { return sizeof(cntk_amd::QuantizedColumn<float>) == 12 ? 0 : 1; }\n' % os.path.join(
        ROOT, "cntk_amd", "cpp", "AllReduceDistGradAggregator.h")
    res = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(rocm, "include"),
                          "-x", "c++", "-"], input=src, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
