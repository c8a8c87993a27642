import importlib
import os
import sys

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO not in sys.path:
    sys.path.insert(0, REPO)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionfinish(session, exitstatus):
    # per-label fp16 parity figures of this run (worst error, elements over a bare 2e-3)
    import json
    from tolerances import FP16_REPORT
    if FP16_REPORT:
        out = os.path.join(REPO, "gpurun_out")
        os.makedirs(out, exist_ok=True)
        path = os.path.join(out, "parity_fp16.json")
        merged = {}
        try:  # a run of part of the suite keeps the other labels of an earlier run
            with open(path) as f:
                merged = json.load(f)
        except (OSError, ValueError):
            pass
        merged.update(FP16_REPORT)
        with open(path, "w") as f:
            json.dump(merged, f, indent=1, sort_keys=True)


def _product():
    return importlib.import_module("mobile-stable-diffusion_amd")


@pytest.fixture(autouse=True)
def _gn_fallbacks_start_at_zero(request):
    """Results that are promised bit for bit hold while no GroupNorm workgroup gave up waiting
    for a sibling (msd_gn_fallbacks() == 0).  Every GPU test starts with the counter at zero, so
    that a failing test's report (below) can say whether that happened during the test."""
    if request.node.get_closest_marker("gpu") is not None:
        try:
            import torch
            if torch.cuda.is_available():
                _product().gn_fallbacks(reset=True)
        except Exception:
            pass
    yield


@pytest.hookimpl(hookwrapper=True)
def pytest_runtest_makereport(item, call):
    outcome = yield
    report = outcome.get_result()
    if report.when == "call" and report.failed and item.get_closest_marker("gpu") is not None:
        try:
            count = _product().gn_fallbacks()
            report.sections.append(("msd_gn_fallbacks", "workgroups that computed a sibling's statistics themselves "
                                    "during this test (current stream and the fixed scratch): %d" % count))
        except Exception as exc:  # the device may be what failed
            report.sections.append(("msd_gn_fallbacks", "not readable: %r" % (exc,)))


@pytest.fixture(scope="session")
def msd():
    """The product package (ctypes access to the HIP library); raises if it is not built."""
    mod = importlib.import_module("mobile-stable-diffusion_amd")
    mod.load_library()
    return mod


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    from oracle import pyoracle
    pyoracle.lib()
    return pyoracle


@pytest.fixture(scope="session")
def golden():
    return np.load(os.path.join(REPO, "tests", "golden", "fixtures.npz"))


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    return torch.device("cuda:0")
