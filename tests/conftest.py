import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    path = os.path.join(ROOT, "tests", "golden", "reference_unit_tests.npz")
    with np.load(path, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def pytest_sessionfinish(session, exitstatus):
    """After a run that made parity checks on a GPU: the measured errors of every check, as
    JSON, next to the other results of the run (tests/parity_report.py turns it into a table)."""
    from tests import parity
    if not parity.REPORT:
        return
    try:
        import torch
        if not torch.cuda.is_available():
            return
    except Exception:
        return
    import json
    out_dir = os.path.join(ROOT, "gpurun_out")
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "parity_report.json"), "w") as f:
        json.dump(parity.REPORT, f, indent=1)
