import os
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
for p in (HERE, ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    return np.load(os.path.join(HERE, "golden", "ref_vectors.npz"), allow_pickle=False)


@pytest.fixture(scope="session")
def golden_fp16_native():
    """Outputs of the reference's avx512fp16 reduce (tests/golden/make_golden.py avx512fp16); inputs of the
    non-grid cases are the float16 inputs of ref_vectors.npz."""
    import numpy as np
    return np.load(os.path.join(HERE, "golden", "ref_vectors_avx512fp16.npz"), allow_pickle=False)


@pytest.fixture(scope="session")
def probes():
    import json
    with open(os.path.join(HERE, "golden", "reference_probes.json")) as f:
        return json.load(f)
