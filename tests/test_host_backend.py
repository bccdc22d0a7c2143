"""The C++ host side: the nGraph-compatible graph / builder / runtime subset and the "HIP" backend
plugin.  The C++ test program (tests/cpp, built into ngraph_amd/host/hip_backend_tests) holds the
reference's own backend tests re-typed; this file runs it."""
import ctypes
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "ngraph_amd", "host")
TESTS = os.path.join(HOST, "hip_backend_tests")


def _run(flag):
    assert os.path.exists(TESTS), "build the host first: make -C ngraph_amd/host"
    p = subprocess.run([TESTS, flag], capture_output=True, text=True, timeout=600)
    print(p.stdout[-6000:])
    print(p.stderr[-2000:])
    assert p.returncode == 0, "C++ tests failed:\n" + "\n".join(l for l in p.stdout.splitlines() if "FAIL" in l)
    return p.stdout


def test_cpp_cpu_suite():
    """type_prop validation, builders + constant folding, plugin discovery, HostTensor"""
    out = _run("--cpu")
    assert "0 failures" in out


def test_plugin_exports_register_symbol():
    """the one C symbol BackendManager looks up with dlsym (backend_manager.cpp:106-113)"""
    lib = ctypes.CDLL(os.path.join(HOST, "libhip_backend.so"), mode=ctypes.RTLD_GLOBAL)
    assert hasattr(lib, "ngraph_register_hip_backend")


@pytest.mark.gpu
def test_cpp_gpu_suite():
    """api / validate_call / unhandled_op, quantized_convolution, quantized_dot, the 28
    quantize_dequantize vectors and the builder_quantization tests, on backend "HIP" """
    out = _run("--gpu")
    assert "0 failures" in out
