import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    # Tests marked gpu are skipped (not failed) when no device is visible and they were not
    # explicitly selected with -m gpu.
    import torch
    if torch.cuda.is_available():
        return
    selected = config.getoption("-m") or ""
    if "gpu" in selected and "not gpu" not in selected:
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def dev():
    import torch
    assert torch.cuda.is_available(), "gpu test selected but no GPU visible"
    return torch.device("cuda:0")


def pytest_terminal_summary(terminalreporter):
    """Observed worst cases of the MLP parity checks of this run (the tolerance they are held to is calibrated
    on the CPU; these are the figures of the HIP path)."""
    mod = sys.modules.get("test_gpu_ccm")
    obs = getattr(mod, "OBSERVED", None) if mod else None
    if obs:
        terminalreporter.write_line(
            f"MLP parity, {len(obs)} comparisons, {sum(o[0] for o in obs)} elements: worst relative error norm "
            f"{max(o[1] for o in obs):.3e}, rows with an element beyond 1e-3*max|ref| + 2 ulp: {sum(o[2] for o in obs)}, "
            f"largest error {max(o[3] for o in obs):.3e} of max|ref|")
