import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def pytest_sessionfinish(session, exitstatus):
    """With CGTP_PARITY_REPORT=<file>: one line per comparison made through helpers.assert_close — test, quantity,
    tolerance, worst element-wise ratio |a-b| / (1 + |b|), worst norm-wise ratio max|a-b| / max(1, max|b|), and, where
    the comparison was given the reference computation restated in fp32 arithmetic, that restatement's own worst
    element-wise ratio against the float64 reference."""
    path = os.environ.get("CGTP_PARITY_REPORT")
    if not path:
        return
    from helpers import PARITY_LOG
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "w") as f:
        f.write("test\twhat\ttol\telementwise\tnormwise\tfp32_reference_elementwise\n")
        for test, what, tol, elem, normwise, ref_elem in PARITY_LOG:
            ref = "" if ref_elem is None else f"{ref_elem:.3e}"
            f.write(f"{test}\t{what}\t{tol:.0e}\t{elem:.3e}\t{normwise:.3e}\t{ref}\n")
