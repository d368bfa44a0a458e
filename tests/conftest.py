import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle; built on demand (gcc only, no GPU needed)."""
    import subprocess
    so = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    from oracle import cpu_ref
    return cpu_ref


@pytest.fixture(scope="session")
def hand_cases():
    """Committed known answers for the literal arrays of the reference's convolution tests
    (tests/golden/reference_hand_cases.json, written by tests/golden/make_hand_cases.py)."""
    import json
    import numpy as np
    with open(os.path.join(ROOT, "tests", "golden", "reference_hand_cases.json")) as f:
        data = json.load(f)
    for case in data["cases"]:
        for key in ("x", "w", "y", "bias_matrix", "y_plus_bias_matrix"):
            if key in case:
                case[key] = np.array(case[key], dtype=np.float32)
    return data["cases"]
