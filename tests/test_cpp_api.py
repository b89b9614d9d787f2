"""The installable C++ API: include/torchscatter/scatter.h + the CMake package.

The reference installs csrc/scatter.h and a TorchScatter CMake package
(CMakeLists.txt:29-78, README.md:156-168). These tests check that this
repository's header declares the same functions and that the operator library
exports them, that the CMake project configures for gfx950, and (on a GPU)
that a consumer program written against the header computes the right thing.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "torchscatter", "scatter.h")
OPLIB = os.path.join(ROOT, "pytorch_scatter_amd", "_torch_scatter_hip.so")
CONSUMER = os.path.join(ROOT, "tests", "cpp_api", "build", "consumer")

# the functions of the reference's C++ API header (csrc/scatter.h:13-80)
API = ["scatter_sum", "scatter_mul", "scatter_mean", "scatter_min", "scatter_max",
       "segment_sum_coo", "segment_mean_coo", "segment_min_coo", "segment_max_coo", "gather_coo",
       "segment_sum_csr", "segment_mean_csr", "segment_min_csr", "segment_max_csr", "gather_csr"]


def test_header_declares_the_reference_api():
    text = open(HEADER).read()
    for name in API:
        assert re.search(r"\b%s\(" % name, text), name
    assert "cuda_version() noexcept" in text


def test_operator_library_exports_the_api():
    if not os.path.exists(OPLIB):
        pytest.skip("operator library not built")
    out = subprocess.run(["nm", "-DC", "--defined-only", OPLIB], capture_output=True, text=True, check=True).stdout
    for name in API:
        assert re.search(r" T %s\(at::Tensor" % name, out), name
    assert " T scatter::cuda_version()" in out


def test_consumer_links_and_reports_version():
    if not os.path.exists(CONSUMER):
        pytest.skip("tests/cpp_api/build/consumer not built (make -C tests/cpp_api)")
    out = subprocess.run([CONSUMER, "--version"], capture_output=True, text=True, timeout=120, check=True).stdout
    assert int(out) > 60000000   # HIP_VERSION = major * 10^7 + ...


@pytest.mark.skipif(shutil.which("cmake") is None, reason="cmake not installed")
def test_cmake_project_configures(tmp_path):
    import torch
    r = subprocess.run(["cmake", "-S", ROOT, "-B", str(tmp_path), "-DCMAKE_PREFIX_PATH=" + torch.utils.cmake_prefix_path],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    cache = open(tmp_path / "CMakeCache.txt").read()
    assert "CMAKE_HIP_ARCHITECTURES:STRING=gfx950" in cache


@pytest.mark.gpu
def test_consumer_program_on_gpu():
    assert os.path.exists(CONSUMER), "tests/cpp_api/build/consumer not built (make -C tests/cpp_api)"
    r = subprocess.run([CONSUMER], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), r.stdout + r.stderr
