"""The C++ host side: the nGraph-compatible graph / builder / runtime subset and the "HIP" backend
plugin.  The C++ test program (tests/cpp, built into ngraph_amd/host/hip_backend_tests) holds the
reference's own backend tests re-typed; every C++ test is one pytest item here, so a failure names
the C++ test that failed."""
import ctypes
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "ngraph_amd", "host")
TESTS = os.path.join(HOST, "hip_backend_tests")


def _listed(kind):
    """names of the C++ tests of one kind ("cpu" / "gpu"); needs no device"""
    if not os.path.exists(TESTS):
        return ["<hip_backend_tests is not built: make -C ngraph_amd/host>"]
    out = subprocess.run([TESTS, "--list"], capture_output=True, text=True, timeout=60).stdout
    return [l.split()[1] for l in out.splitlines() if l.startswith(kind + " ")]


def _run(flag, name):
    assert os.path.exists(TESTS), "build the host first: make -C ngraph_amd/host"
    print("[case] hip_backend_tests", flag, name, flush=True)
    p = subprocess.run([TESTS, flag, "--exact", name], capture_output=True, text=True, timeout=600)
    print(p.stdout[-6000:])
    print(p.stderr[-2000:])
    assert p.returncode == 0, "C++ test %s failed (exit %d):\n%s" % (
        name, p.returncode, "\n".join(l for l in p.stdout.splitlines() if "FAIL" in l))
    assert "1 tests ran, 0 failures" in p.stdout


@pytest.mark.parametrize("name", _listed("cpu"))
def test_cpp_cpu(name):
    """type_prop validation, builders + constant folding, plugin discovery, HostTensor"""
    _run("--cpu", name)


def test_plugin_exports_register_symbol():
    """the one C symbol BackendManager looks up with dlsym (backend_manager.cpp:106-113)"""
    lib = ctypes.CDLL(os.path.join(HOST, "libhip_backend.so"), mode=ctypes.RTLD_GLOBAL)
    assert hasattr(lib, "ngraph_register_hip_backend")


def test_plugin_sources_compile_against_reference_headers():
    """hip_backend.cpp and the fusion pass are written against the real nGraph API: `make refcheck`
    compiles them (syntax only) with the reference tree's headers first on the include path.  The
    reference tree exists only where this build was made; elsewhere there is nothing to check."""
    ref = "/root/reference"
    if not os.path.isdir(os.path.join(ref, "src", "ngraph")):
        pytest.skip("no nGraph source tree at " + ref)
    p = subprocess.run(["make", "-C", HOST, "refcheck", "REF=" + ref], capture_output=True, text=True, timeout=600)
    print(p.stdout[-3000:])
    print(p.stderr[-3000:])
    assert p.returncode == 0 and "refcheck ok" in p.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("name", _listed("gpu"))
def test_cpp_gpu(name):
    """api / validate_call / unhandled_op, quantized_convolution, quantized_dot, the 28
    quantize_dequantize vectors, the builder_quantization tests, fusion, layout, ResNet-50, on
    backend "HIP" """
    _run("--gpu", name)
