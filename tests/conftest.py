import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _backward_error_word(request):
    """Every GPU test reads the error word of each backward it runs (the word a kernel sets when it
    abandons one of its bounded internal waits) and fails if it is set: a give-up would otherwise
    hand back wrong gradients with return code 0."""
    if "gpu" not in request.keywords:
        yield
        return
    from flame_amd import _lib
    _lib.check_gave_up(True)
    try:
        yield
    finally:
        _lib.check_gave_up(None)


def pytest_sessionfinish(session, exitstatus):
    """SBA_MARGINS_FILE=<path>: error / tolerance of every parity check made through helpers.within()."""
    path = os.environ.get("SBA_MARGINS_FILE")
    if not path:
        return
    import helpers
    worst = {}
    for label, quantity, err, tol in helpers.MARGINS:
        key = (label, quantity)
        if key not in worst or err / tol > worst[key][0] / worst[key][1]:
            worst[key] = (err, tol)
    labels = sorted({k[0] for k in worst}, key=lambda lab: -max(e / t for (l, _), (e, t) in worst.items() if l == lab))
    with open(path, "w") as f:
        f.write("check                                                              quantity    error   tolerance  error/tolerance\n")
        for lab in labels:
            for (l, q), (e, t) in sorted(worst.items()):
                if l == lab:
                    f.write(f"{lab:66s} {q:8s} {e:10.3e} {t:9.1e} {e / t:8.3f}\n")
