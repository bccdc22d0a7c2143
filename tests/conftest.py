import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def kats():
    with open(os.path.join(GOLDEN, "reference_kats.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def qdq_kats():
    with open(os.path.join(GOLDEN, "quantize_dequantize_kats.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def ref_vectors():
    with open(os.path.join(GOLDEN, "ref_vectors.json")) as f:
        manifest = json.load(f)
    arrays = np.load(os.path.join(GOLDEN, "ref_vectors.npz"))
    return manifest, arrays


@pytest.fixture(scope="session")
def gpu_lib():
    """libhipq.so on a machine with a GPU; fails (never skips) if the library is missing."""
    from ngraph_amd import hipq as H

    lib = H.load()
    n = H.C.c_int(0)
    H.check(lib.hipq_device_count(H.C.byref(n)))
    assert n.value >= 1, "no HIP device visible"
    H.check(lib.hipq_set_device(0))
    return lib
